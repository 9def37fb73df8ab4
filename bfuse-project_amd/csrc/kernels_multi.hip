// Fusions of three and four operators -- the reference's emitter takes a list of kernels of any
// length (horizontal-fuser/src/Algorithms.cc:23-35,540-566).  Small instances for the parity
// tests (their standalone kernels are defined with the other small instances), and one full-size
// group: the fp32 QKV projection, the LayerNorm and the causal softmax of one transformer layer.
#include "fuse.h"
#include "ops_conv.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_pool.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// the same instantiations the small standalone kernels are built from
using GemmS2 = GemmF32<96, 192, 128, 32, 64, 2, kEpiGeluTanh, 3>;     // 9 tiles x 128 threads, barriers
using GemmS5 = GemmF32Dma<128, 192, 160, 32, 96, 2>;                  // 8 tiles x 128 threads, barriers
using BiasReluS = BiasRelu<4096, 64, 4>;                              // 16 blocks x 64 threads
using LayerNormS = LayerNorm<8, 256, 2, 1>;                           
using SoftmaxS = SoftmaxCausal<2, 256, 2, 2, 2>;
using ConvS2 = Conv3x3F32Lds<32, 32, 12, 12, 16, 1, 2>;               // 18 tiles x 128 threads, barriers
using PoolS = MaxPool3x3S2<4, 16, 16, 64>;

// block fusion of three: every pattern (unequal grids, unequal block widths, two barrier-bearing sides)
BFUSE_BFUSE3_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS, , bfuse::kZigzag, 2, 1)
BFUSE_BFUSE3_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS, _p2, bfuse::kProportional, 2, 1)
BFUSE_BFUSE3_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS, _c4, bfuse::kChunked, 4, 1)
BFUSE_BFUSE3_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS, _r, bfuse::kRanges, 0, 0)
// four operators
BFUSE_BFUSE4_KERNEL(gemm_f32_128x160x192_d, GemmS5, layernorm_8x256, LayerNormS, softmax_causal_2x256x256, SoftmaxS, maxpool3x3s2_f32_4x16x16, PoolS, _c2, bfuse::kChunked, 2, 1)
BFUSE_BFUSE4_KERNEL(gemm_f32_128x160x192_d, GemmS5, layernorm_8x256, LayerNormS, softmax_causal_2x256x256, SoftmaxS, maxpool3x3s2_f32_4x16x16, PoolS, , bfuse::kZigzag, 1, 1)
// run-time plan and persistent workgroups over three operators
BFUSE_BFUSE_RT3_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS)

// thread-level fusion of three: one synchronising side keeps the hardware barrier ...
BFUSE_HFUSE3_KERNEL(gemm_f32_128x160x192_d, GemmS5, bias_relu_4096, BiasReluS, maxpool3x3s2_f32_4x16x16, PoolS)
// ... two synchronising sides get an LDS arrival counter each, the third has none
BFUSE_HFUSE3_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS)
// four sides in one workgroup (128 + 128 + 64 + 64 threads)
BFUSE_HFUSE4_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_f32_128x160x192_d, GemmS5, layernorm_8x256, LayerNormS, bias_relu_4096, BiasReluS)

// Full size: QKV projection 512x768x2304 (256 tiles, MFMA-bound), LayerNorm 512x768 and causal
// softmax 12x512x512 (memory-bound), the kernels of pairs 2 and 4.  The GEMM runs here with a ring
// of two stages: every workgroup of a block-fused kernel is charged the largest side's LDS, and
// with 48 KB instead of 72 three workgroups fit a CU instead of two -- the GEMM alone is as fast
// (16.0 us either way), the fused kernel 19.0 instead of 20.6 us.
using GemmQkvS2 = GemmF32Dma<512, 2304, 768, 32, 144, 4, kEpiNone, 2>;
using LnBert = LayerNorm<512, 768, 1, 1>;
using Softmax4 = SoftmaxCausal<12, 512, 4, 1>;
BFUSE_KERNEL(gemm_f32_512x768x2304_s2, GemmQkvS2, ({{512, 768, 1, 1}, 4}), ({{768, 2304, 1, 1}, 4}), ({{512, 2304, 1, 1}, 4}))
// GEMM tiles first (one per CU), then the two memory-bound grids in their shadow
BFUSE_BFUSE3_KERNEL(gemm_f32_512x768x2304_s2, GemmQkvS2, layernorm_512x768, LnBert, softmax_causal_12x512x512, Softmax4, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE3_KERNEL(gemm_f32_512x768x2304_s2, GemmQkvS2, layernorm_512x768, LnBert, softmax_causal_12x512x512, Softmax4, _r, bfuse::kRanges, 0, 0)
BFUSE_BFUSE_RT3_KERNEL(gemm_f32_512x768x2304_s2, GemmQkvS2, layernorm_512x768, LnBert, softmax_causal_12x512x512, Softmax4)
