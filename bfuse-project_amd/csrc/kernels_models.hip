// Further dense layers of the reference's example models (test-utils/examples/llm.yaml:7-41), beyond the
// ones the five benchmark configurations use: the same fp32 and bf16 GEMM templates at other shapes, so that the ids
// of that file resolve to kernels of the library (bfuse_project_amd.configure).  Tiles are chosen as one per
// CU (256 workgroups) where the shape allows it.
#include "fuse.h"
#include "ops_conv.h"
#include "ops_gemm_bf16.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// dense_0: BERT attention output projection, [512 x 768] . [768 x 768]: 16 x 16 tiles of 32 x 48
using Dense0 = GemmF32Dma<512, 768, 768, 32, 48, 4>;
// dense_1: BERT / GPT-2 MLP up-projection without the activation, [512 x 768] . [768 x 3072]: pair 4's tiling
using Dense1 = GemmF32Dma<512, 3072, 768, 32, 96, 4, kEpiNone, 2>;
// dense_2: MLP down-projection, [512 x 3072] . [3072 x 768]
using Dense2 = GemmF32Dma<512, 768, 3072, 32, 48, 4>;
// dense_5: Llama-3-8B key / value projection, [512 x 4096] . [4096 x 1024]: 16 x 16 tiles of 32 x 64
using Dense5 = GemmF32Dma<512, 1024, 4096, 32, 64, 4>;

BFUSE_KERNEL(gemm_f32_512x768x768, Dense0, ({{512, 768, 1, 1}, 4}), ({{768, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_512x768x3072, Dense1, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_512x3072x768, Dense2, ({{512, 3072, 1, 1}, 4}), ({{3072, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_512x4096x1024, Dense5, ({{512, 4096, 1, 1}, 4}), ({{4096, 1024, 1, 1}, 4}), ({{512, 1024, 1, 1}, 4}))

// each with the LayerNorm of pair 2 as its memory-bound partner, block-fused one chunk per round over the CUs
using LayerNormW1 = LayerNorm<512, 768, 1, 1>;
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x768, Dense0, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x3072, Dense1, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x3072x768, Dense2, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x4096x1024, Dense5, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)

// Llama-3-8B, bf16 as pair 5's GEMM, weights [N, K]: dense_4 (query / output projection,
// [512 x 4096] . [4096 x 4096]^T) and dense_7 (MLP down-projection, [512 x 14336] . [4096 x 14336]^T).
// N = 4096 over 256 CUs leaves each a 64 x 128 tile: four compute waves (2 x 2) of 32 x 64 and two
// producer waves, ring of three 64-k stages (72 KB), read-ahead of two fragments, the next step's barrier
// before MFMA group 6 of 8.
using Dense4 = GemmBf16NTDma<512, 4096, 4096, 64, 128, 3, 2, 2, 2, 2, 6>;
using Dense7 = GemmBf16NTDma<512, 4096, 14336, 64, 128, 3, 2, 2, 2, 2, 6>;
BFUSE_KERNEL(gemm_bf16_512x4096x4096, Dense4, ({{512, 4096, 1, 1}, 2}), ({{4096, 4096, 1, 1}, 2}), ({{512, 4096, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, ({{512, 14336, 1, 1}, 2}), ({{4096, 14336, 1, 1}, 2}), ({{512, 4096, 1, 1}, 2}))
// each with pair 5's RMSNorm + RoPE side (one row per one-wave workgroup), block-fused one chunk per round
using NormRopeW1 = RmsNormRope<512, 32, 128, 1>;
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x4096, Dense4, rmsnorm_rope_bf16_512x4096, NormRopeW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, rmsnorm_rope_bf16_512x4096, NormRopeW1, _c256, bfuse::kChunked, 256, 1)

// ResNet-18 (test-utils/examples/resnet-18.yaml): conv2d_4, the second 3x3 / stride 1 / padding 1 convolution the
// template's row alignment allows (128 -> 128 channels on 28 x 28): 32 output channels x 16 pixels per workgroup,
// four waves take two 16-channel groups each, 49 x 4 = 196 workgroups
using Conv128 = Conv3x3F32Lds<128, 128, 28, 28, 32, 1, 4>;
BFUSE_KERNEL(conv3x3_f32_128x28x28_128, Conv128, ({{1, 128, 28, 28}, 4}), ({{128, 128, 3, 3}, 4}), ({{1, 128, 28, 28}, 4}))
BFUSE_BFUSE_KERNEL(conv3x3_f32_128x28x28_128, Conv128, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)

// Batched GEMMs of the attention layers (the reference's bgemm, scripts/configure_kernels.py:14-19,40-48:
// C[b] = A[b] . B[b]^T with A [b, M, K] and B [b, N, K]): bgemm_0 / bgemm_1 are BERT's and GPT-2's scores and
// context products (12 heads, sequence 512, head size 64), bgemm_2 / bgemm_3 Llama-3-8B's (32 heads, head size 128).
// Operands go global -> VGPR in MFMA layout (both are contiguous along K); a short reduction (K = 64, 128) is
// one wave's, a long one (K = 512) is split over two.
// (tiles measured on bgemm_0 / bgemm_1: 64 x 64 one-wave 8.0 us, 32 x 64 8.3-9.0, 32 x 128 8.0, 16 x 64 10.1, 64 x 128 11.1;
//  32 x 64 two-wave 9.7 us, 16 x 64 two-wave 11.3, four-wave 11.3, 16 x 32 10.1)
using Bgemm0 = GemmF32<512, 512, 64, 64, 64, 1, kEpiNone, 2, 1, true, 12>;     // 8 x 8 tiles x 12 = 768 one-wave workgroups
using Bgemm1 = GemmF32<512, 64, 512, 32, 64, 2, kEpiNone, 2, 1, true, 12>;     // 16 x 1 tiles x 12 = 192 two-wave workgroups
using Bgemm2 = GemmF32<512, 512, 128, 64, 64, 1, kEpiNone, 2, 1, true, 32>;    // 2048 one-wave workgroups
using Bgemm3 = GemmF32<512, 128, 512, 32, 64, 2, kEpiNone, 2, 1, true, 32>;    // 16 x 2 tiles x 32 = 1024 two-wave workgroups
BFUSE_KERNEL(bgemm_f32_12x512x64x512, Bgemm0, ({{12, 512, 64, 1}, 4}), ({{12, 512, 64, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_12x512x512x64, Bgemm1, ({{12, 512, 512, 1}, 4}), ({{12, 64, 512, 1}, 4}), ({{12, 512, 64, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_32x512x128x512, Bgemm2, ({{32, 512, 128, 1}, 4}), ({{32, 512, 128, 1}, 4}), ({{32, 512, 512, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_32x512x512x128, Bgemm3, ({{32, 512, 512, 1}, 4}), ({{32, 128, 512, 1}, 4}), ({{32, 512, 128, 1}, 4}))
// the scores product of BERT / GPT-2 with the causal softmax that follows it in the model as its partner,
// and with the LayerNorm
using Softmax4W = SoftmaxCausal<12, 512, 4, 1>;
BFUSE_BFUSE_KERNEL(bgemm_f32_12x512x64x512, Bgemm0, softmax_causal_12x512x512, Softmax4W, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(bgemm_f32_12x512x512x64, Bgemm1, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
