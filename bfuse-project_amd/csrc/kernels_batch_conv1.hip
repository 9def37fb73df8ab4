// Batch-1024 convolutions of the reference's example configurations (test-utils/examples/benchmark.yaml,
// inception_v3.yaml; argument lists N, H, W, CO, CI, KH, KW, stride, padding) on the general convolutions (64 consecutive pixels or a
// 4 x 16 rectangle per workgroup) with the library's default tiling.  Names: conv<KH>x<KW>s<stride>p<padding>_f32_<N>x<CI>x<H>x<W>_<CO>.  Part 1 of 4.
#include "fuse.h"
#include "ops_conv_rect.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

#define CONV_BATCH(N, CI, H, W, CO, KH, KW, S, P)                                                                 \
    using Conv_##N##_##CI##_##H##_##W##_##CO##_##KH##_##KW##_##S##_##P = ConvF32Auto<CI, CO, H, W, KH, KW, S, P, N>; \
    BFUSE_KERNEL(conv##KH##x##KW##s##S##p##P##_f32_##N##x##CI##x##H##x##W##_##CO,                                    \
                 Conv_##N##_##CI##_##H##_##W##_##CO##_##KH##_##KW##_##S##_##P, ({{N, CI, H, W}, 4}), ({{CO, CI, KH, KW}, 4}), \
                 ({{N, CO, (H - KH + 2 * P) / S + 1, (W - KW + 2 * P) / S + 1}, 4}))

CONV_BATCH(1024, 3, 224, 224, 64, 7, 7, 2, 3)
CONV_BATCH(1024, 128, 28, 28, 128, 3, 3, 1, 1)
CONV_BATCH(1024, 128, 28, 28, 256, 1, 1, 2, 0)
CONV_BATCH(1024, 256, 35, 35, 64, 1, 1, 1, 0)
CONV_BATCH(1024, 288, 35, 35, 384, 3, 3, 2, 0)
CONV_BATCH(1024, 768, 17, 17, 160, 1, 1, 1, 0)
CONV_BATCH(1024, 32, 147, 147, 64, 3, 3, 1, 1)
CONV_BATCH(1024, 192, 35, 35, 48, 1, 1, 1, 0)
CONV_BATCH(1024, 192, 35, 35, 32, 1, 1, 1, 0)
CONV_BATCH(1024, 448, 8, 8, 384, 3, 3, 1, 1)
CONV_BATCH(1024, 2048, 8, 8, 448, 1, 1, 1, 0)
