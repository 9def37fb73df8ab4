// Batch-1024 convolutions of the reference's third generated suite (tests/interleave_scheduler/config/info.yaml;
// argument lists N, H, W, CO, CI, KH, KW, stride, padding) on the general convolutions (64 consecutive pixels or a
// 4 x 16 rectangle per workgroup) with the library's default tiling.  Names: conv<KH>x<KW>s<stride>p<padding>_f32_<N>x<CI>x<H>x<W>_<CO>.
#include "fuse.h"
#include "ops_conv_rect.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

#define CONV_BATCH(N, CI, H, W, CO, KH, KW, S, P)                                                                 \
    using Conv_##N##_##CI##_##H##_##W##_##CO##_##KH##_##KW##_##S##_##P = ConvF32Auto<CI, CO, H, W, KH, KW, S, P, N>; \
    BFUSE_KERNEL(conv##KH##x##KW##s##S##p##P##_f32_##N##x##CI##x##H##x##W##_##CO,                                    \
                 Conv_##N##_##CI##_##H##_##W##_##CO##_##KH##_##KW##_##S##_##P, ({{N, CI, H, W}, 4}), ({{CO, CI, KH, KW}, 4}), \
                 ({{N, CO, (H - KH + 2 * P) / S + 1, (W - KW + 2 * P) / S + 1}, 4}))

CONV_BATCH(1024, 64, 112, 112, 192, 3, 3, 2, 0)
CONV_BATCH(1024, 32, 147, 147, 64, 3, 3, 2, 0)
CONV_BATCH(1024, 64, 56, 56, 128, 3, 3, 1, 0)
CONV_BATCH(1024, 128, 28, 28, 256, 3, 3, 1, 0)
CONV_BATCH(1024, 16, 227, 227, 64, 3, 3, 4, 0)
CONV_BATCH(1024, 256, 56, 56, 256, 1, 1, 1, 0)
