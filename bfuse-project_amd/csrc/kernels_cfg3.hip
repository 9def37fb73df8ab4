// Pair 3 (ResNet-18 shapes): 3x3 conv, stride 1, pad 1, NCHW [1,64,56,56] -> 64 channels,
// zig-zag block-fused with a 3x3 stride-2 max-pool on [1,64,112,112].
#include "fuse.h"
#include "ops_conv.h"
#include "ops_pool.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// 16 output channels x 64 pixels per workgroup; four waves take one 16-channel group each
using Conv64 = Conv3x3F32Lds<64, 64, 56, 56, 16, 4, 4>;    // 4 x 49 = 196 workgroups, 74 KB
using Pool = MaxPool3x3S2<64, 112, 112, 256>;              // 196 workgroups

BFUSE_KERNEL(conv3x3_f32_64x56x56_64, Conv64, ({{1, 64, 56, 56}, 4}), ({{64, 64, 3, 3}, 4}), ({{1, 64, 56, 56}, 4}))
BFUSE_KERNEL(maxpool3x3s2_f32_64x112x112, Pool, ({{1, 64, 112, 112}, 4}), ({{1, 1, 1, 1}, 4}), ({{1, 64, 56, 56}, 4}))

BFUSE_BFUSE_KERNEL(conv3x3_f32_64x56x56_64, Conv64, maxpool3x3s2_f32_64x112x112, Pool, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(conv3x3_f32_64x56x56_64, Conv64, maxpool3x3s2_f32_64x112x112, Pool, _c8, bfuse::kChunked, 8, 1)
BFUSE_BFUSE_KERNEL(conv3x3_f32_64x56x56_64, Conv64, maxpool3x3s2_f32_64x112x112, Pool, _c256, bfuse::kChunked, 256, 1)
BFUSE_HFUSE_KERNEL(conv3x3_f32_64x56x56_64, Conv64, maxpool3x3s2_f32_64x112x112, Pool)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(conv3x3_f32_64x56x56_64, Conv64, maxpool3x3s2_f32_64x112x112, Pool)
