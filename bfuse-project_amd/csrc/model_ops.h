// The operators of the reference's example models as the library instantiates them: one alias per operator id
// (test-utils/examples/llm.yaml, resnet-18.yaml).  A fused kernel and the standalone kernel it is compared
// with must be built from the SAME instantiation, so every file that names one of these takes it from here.
#pragma once
#include "ops_conv.h"
#include "ops_gemm_bf16.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_rowwise.h"

namespace bfuse {
namespace model {

// dense_0: BERT attention output projection, [512 x 768] . [768 x 768]: 16 x 16 tiles of 32 x 48
using Dense0 = GemmF32Dma<512, 768, 768, 32, 48, 4>;
// dense_1: BERT / GPT-2 MLP up-projection without the activation, [512 x 768] . [768 x 3072]: pair 4's tiling
using Dense1 = GemmF32Dma<512, 3072, 768, 32, 96, 4, kEpiNone, 2>;
// dense_2: MLP down-projection, [512 x 3072] . [3072 x 768]
using Dense2 = GemmF32Dma<512, 768, 3072, 32, 48, 4>;
// dense_3: the QKV projection of pair 2
using Dense3 = GemmF32Dma<512, 2304, 768, 32, 144, 4>;
// dense_4 / dense_7 (Llama-3-8B, bf16, weights [N, K]): N = 4096 over 256 CUs leaves each a 64 x 128 tile: four
// compute waves (2 x 2) of 32 x 64 and two producer waves, ring of three 64-k stages (72 KB), read-ahead of two
// fragments, the next step's barrier before MFMA group 6 of 8
using Dense4 = GemmBf16NTDma<512, 4096, 4096, 64, 128, 3, 2, 2, 2, 2, 6>;
using Dense7 = GemmBf16NTDma<512, 4096, 14336, 64, 128, 3, 2, 2, 2, 2, 6>;
// dense_5: Llama-3-8B key / value projection, [512 x 4096] . [4096 x 1024]: 16 x 16 tiles of 32 x 64
using Dense5 = GemmF32Dma<512, 1024, 4096, 32, 64, 4>;
// dense_6: the gate projection of pair 5
using Dense6 = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4, 4, 2, 2, 11>;

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

// conv2d_1: the convolution of pair 3;  conv2d_4: 128 -> 128 channels on 28 x 28, 32 output channels x 16 pixels
// per workgroup, four waves take two 16-channel groups each, 49 x 4 = 196 workgroups
using Conv1 = Conv3x3F32Lds<64, 64, 56, 56, 16, 4, 4>;
using Conv4 = Conv3x3F32Lds<128, 128, 28, 28, 32, 1, 4>;

// memory-bound partners
using LayerNormW1 = LayerNorm<512, 768, 1, 1>;
using NormRopeW1 = RmsNormRope<512, 32, 128, 1>;
using Softmax4W = SoftmaxCausal<12, 512, 4, 1>;

}  // namespace model
}  // namespace bfuse
