// The operators of the reference's example models as the library instantiates them: one alias per operator id
// (test-utils/examples/llm.yaml, resnet-18.yaml).  A fused kernel and the standalone kernel it is compared
// with must be built from the SAME instantiation, so every file that names one of these takes it from here.
#pragma once
#include "ops_conv.h"
#include "ops_conv_general.h"
#include "ops_conv_rect.h"
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

// fp32 instantiations of the Llama-3-8B layers (the reference computes every layer in fp32): 64 x 128 tiles,
// one per CU for N = 4096 (dense_4, dense_7) and two rounds of them for N = 14336 (dense_6)
using Dense4F32 = GemmF32Dma<512, 4096, 4096, 64, 128, 4>;
using Dense6F32 = GemmF32Dma<512, 14336, 4096, 64, 128, 4>;
using Dense7F32 = GemmF32Dma<512, 4096, 14336, 64, 128, 4>;

// bgemm_4 .. bgemm_17 of llm.yaml (ViT / Swin / small-model attention products: 16 heads x 256 or 208 tokens with
// head sizes 64 and 80, and single-head products of 512 / 768 / 1024 tokens).  208 = 13 x 16 and 80 = 5 x 16 are
// whole 16-wide MFMA blocks: a 208-column tile is three 64-column groups and one of 16, an 80-column tile one of
// each; reductions of 80 and 208 are five and thirteen 16-k stages of one wave.
using Bgemm4 = GemmF32<256, 256, 64, 64, 64, 1, kEpiNone, 2, 1, true, 16>;      // 4 x 4 tiles x 16 = 256 one-wave workgroups
using Bgemm5 = GemmF32<256, 64, 256, 16, 64, 2, kEpiNone, 2, 1, true, 16>;      // 16 x 1 x 16 = 256 two-wave workgroups
using Bgemm6 = GemmF32<256, 256, 80, 64, 64, 1, kEpiNone, 2, 1, true, 16>;
using Bgemm7 = GemmF32<256, 80, 256, 16, 80, 2, kEpiNone, 2, 1, true, 16>;
using Bgemm8 = GemmF32<208, 208, 64, 16, 208, 1, kEpiNone, 2, 1, true, 16>;     // 13 x 1 x 16 = 208 one-wave workgroups
using Bgemm9 = GemmF32<208, 64, 208, 16, 64, 1, kEpiNone, 2, 1, true, 16>;
using Bgemm10 = GemmF32<208, 208, 80, 16, 208, 1, kEpiNone, 2, 1, true, 16>;
using Bgemm11 = GemmF32<208, 80, 208, 16, 80, 1, kEpiNone, 2, 1, true, 16>;
using Bgemm12 = GemmF32<512, 256, 64, 16, 64, 1, kEpiNone, 2, 1, true, 1>;      // 32 x 4 = 128 one-wave workgroups
using Bgemm13 = GemmF32<512, 64, 256, 16, 64, 4, kEpiNone, 2, 1, true, 1>;      // 32 four-wave workgroups
using Bgemm14 = GemmF32<768, 384, 64, 16, 64, 1, kEpiNone, 2, 1, true, 1>;      // 48 x 6 = 288
using Bgemm15 = GemmF32<768, 64, 384, 16, 64, 4, kEpiNone, 2, 1, true, 1>;      // 48 four-wave workgroups
using Bgemm16 = GemmF32<1024, 512, 64, 32, 64, 1, kEpiNone, 2, 1, true, 1>;     // 32 x 8 = 256
using Bgemm17 = GemmF32<1024, 64, 512, 16, 64, 4, kEpiNone, 2, 1, true, 1>;     // 64 four-wave workgroups

// The other ResNet-18 layers (test-utils/examples/resnet-18.yaml) on the general convolution:
// <CI, CO, H, W, KH, KW, stride, padding, output channels per workgroup, 16-pixel blocks, waves>
using Conv0 = ConvF32Rect<3, 64, 224, 224, 7, 7, 2, 3, 16, 4, 1>;         // 7x7 stride 2 on RGB: 4 x 16-pixel rectangles (13 x 37 patch instead of 9 x 230), 196 x 4 = 784 one-wave workgroups
using Conv2 = SwapOperands<GemmF32<64, 3136, 64, 16, 64, 1>>;            // 1x1 stride 1 = Wt[64,64] . X[64,3136]: 4 x 49 = 196
using Conv3 = ConvF32Lds<64, 128, 56, 56, 3, 3, 2, 1, 32, 1, 4>;          // 49 x 4 = 196 workgroups
using Conv5 = ConvF32Lds<64, 128, 56, 56, 1, 1, 2, 0, 32, 1, 4>;
using Conv6 = ConvF32Lds<128, 256, 28, 28, 3, 3, 2, 1, 16, 1, 4>;         // 13 x 16 = 208
using Conv7 = ConvF32Lds<256, 256, 14, 14, 3, 3, 1, 1, 16, 1, 4>;
using Conv8 = ConvF32Lds<128, 256, 28, 28, 1, 1, 2, 0, 16, 1, 4>;
using Conv9 = ConvF32Lds<256, 512, 14, 14, 3, 3, 2, 1, 16, 1, 4>;         // 4 x 32 = 128
using Conv10 = ConvF32Lds<512, 512, 7, 7, 3, 3, 1, 1, 16, 1, 4>;
using Conv11 = ConvF32Lds<256, 512, 14, 14, 1, 1, 2, 0, 16, 1, 4>;

// memory-bound partners
using LayerNormW1 = LayerNorm<512, 768, 1, 1>;
using NormRopeW1 = RmsNormRope<512, 32, 128, 1>;
using Softmax4W = SoftmaxCausal<12, 512, 4, 1>;

}  // namespace model
}  // namespace bfuse
