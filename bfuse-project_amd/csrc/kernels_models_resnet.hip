// The remaining operator ids of the reference's resnet-18.yaml on the general convolution
// (ops_conv_general.h): 7x7 stride 2, 1x1 (stride 1 as a GEMM, stride 2 on the staged patch), 3x3 stride 2,
// and 3x3 on 14x14 and 7x7 images.  Names: conv<KH>x<KW>s<stride>p<padding>_f32_<CI>x<H>x<W>_<CO>.  Each with
// a memory-bound partner, block-fused one chunk per round over the CUs.
#include "fuse.h"
#include "model_ops.h"

using namespace bfuse;
using namespace bfuse::model;

BFUSE_MODULE_PROLOGUE()

#define CONV_F32(NAME, OP, CI, H, W, CO, KH, KW, OH, OW)                                                          \
    BFUSE_KERNEL(NAME, OP, ({{1, CI, H, W}, 4}), ({{CO, CI, KH, KW}, 4}), ({{1, CO, OH, OW}, 4}))                   \
    BFUSE_BFUSE_KERNEL(NAME, OP, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
CONV_F32(conv7x7s2p3_f32_3x224x224_64, Conv0, 3, 224, 224, 64, 7, 7, 112, 112)
CONV_F32(conv1x1s1p0_f32_64x56x56_64, Conv2, 64, 56, 56, 64, 1, 1, 56, 56)
CONV_F32(conv3x3s2p1_f32_64x56x56_128, Conv3, 64, 56, 56, 128, 3, 3, 28, 28)
CONV_F32(conv1x1s2p0_f32_64x56x56_128, Conv5, 64, 56, 56, 128, 1, 1, 28, 28)
CONV_F32(conv3x3s2p1_f32_128x28x28_256, Conv6, 128, 28, 28, 256, 3, 3, 14, 14)
CONV_F32(conv3x3s1p1_f32_256x14x14_256, Conv7, 256, 14, 14, 256, 3, 3, 14, 14)
CONV_F32(conv1x1s2p0_f32_128x28x28_256, Conv8, 128, 28, 28, 256, 1, 1, 14, 14)
CONV_F32(conv3x3s2p1_f32_256x14x14_512, Conv9, 256, 14, 14, 512, 3, 3, 7, 7)
CONV_F32(conv3x3s1p1_f32_512x7x7_512, Conv10, 512, 7, 7, 512, 3, 3, 7, 7)
CONV_F32(conv1x1s2p0_f32_256x14x14_512, Conv11, 256, 14, 14, 512, 1, 1, 7, 7)
