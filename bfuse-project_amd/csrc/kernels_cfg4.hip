// Pair 4 (GPT-2 small shapes, seq 512): causal softmax over 12 x [512x512] fp32 scores
// block-fused with the MLP up-projection GEMM [512x768].[768x3072] fp32 + tanh-GELU.
#include "fuse.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_gemm_f32_lds.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// softmax: one row per wave; 4-wave workgroups (1536), 1-wave workgroups (6144), and a
// 256-workgroup shape (4 waves x 6 rows) whose grid matches the GEMM's for horizontal fusion
using Softmax4 = SoftmaxCausal<12, 512, 4, 1>;
using Softmax1 = SoftmaxCausal<12, 512, 1, 1>;
using Softmax4x6 = SoftmaxCausal<12, 512, 4, 6, 3>;
using Softmax4b = SoftmaxCausal<12, 512, 4, 4, 4>;   // 384 workgroups, 4 rows in flight per wave
// GEMM + GELU: 256 workgroups, four waves split K = 768
using GemmFc = GemmF32<512, 3072, 768, 64, 96, 4, kEpiGeluTanh, 2, 0>;     // 8 x 32 tiles of 64x96
using GemmFcH = GemmF32<512, 3072, 768, 32, 96, 4, kEpiGeluTanh, 2, 0>;    // 32 x 16 tiles of 32x96, two per CU
using GemmFcW = GemmF32<512, 3072, 768, 32, 192, 4, kEpiGeluTanh, 2, 0>;   // 16 x 16 tiles of 32x192


BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(softmax_causal_12x512x512_w1, Softmax1, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(softmax_causal_12x512x512_r6, Softmax4x6, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072, GemmFc, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_h, GemmFcH, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_t32, GemmFcW, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))

BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072, GemmFc, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072, GemmFc, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_w1, Softmax1, gemm_gelu_f32_512x768x3072, GemmFc, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_w1, Softmax1, gemm_gelu_f32_512x768x3072_t32, GemmFcW, _c256, bfuse::kChunked, 256, 1)
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r6, Softmax4x6, gemm_gelu_f32_512x768x3072, GemmFc)
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r6, Softmax4x6, gemm_gelu_f32_512x768x3072_t32, GemmFcW)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, gemm_gelu_f32_512x768x3072, GemmFc, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, gemm_gelu_f32_512x768x3072_h, GemmFcH, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, gemm_gelu_f32_512x768x3072_h, GemmFcH, _c512, bfuse::kChunked, 512, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_h, GemmFcH, _c512, bfuse::kChunked, 512, 1)
// 32x96 tiles with three register stages; softmax as 512 workgroups (4 waves x 3 rows, all in flight)
using GemmFcH3 = GemmF32<512, 3072, 768, 32, 96, 4, kEpiGeluTanh, 3, 0>;
using Softmax4x3 = SoftmaxCausal<12, 512, 4, 3, 3>;
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_h3, GemmFcH3, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_KERNEL(softmax_causal_12x512x512_r3, Softmax4x3, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, gemm_gelu_f32_512x768x3072_h3, GemmFcH3, _c512, bfuse::kChunked, 512, 1)
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r3, Softmax4x3, gemm_gelu_f32_512x768x3072_h, GemmFcH)
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r3, Softmax4x3, gemm_gelu_f32_512x768x3072_h3, GemmFcH3)
// LDS-staged GEMM: 64x96 tiles, eight waves of 16x48, no K split; softmax as 256 workgroups of 4 waves x 6 rows
using GemmFcL = GemmF32Lds<512, 3072, 768, 64, 96, 48, kEpiGeluTanh, 4>;
using Softmax4x6b = SoftmaxCausal<12, 512, 4, 6, 3>;
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_l, GemmFcL, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r6, Softmax4x6, gemm_gelu_f32_512x768x3072_l, GemmFcL)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, gemm_gelu_f32_512x768x3072_l, GemmFcL, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_l, GemmFcL, _c256, bfuse::kChunked, 256, 1)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_l, GemmFcL)
// split-K with per-wave LDS rings
using GemmFcD = GemmF32Dma<512, 3072, 768, 64, 96, 4, kEpiGeluTanh>;
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_d, GemmFcD, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_d, GemmFcD, _c256, bfuse::kChunked, 256, 1)
using GemmFcDh = GemmF32Dma<512, 3072, 768, 32, 96, 4, kEpiGeluTanh>;   // 16 x 32 = 512 tiles of 32 x 96: two workgroups per CU
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_dh, GemmFcDh, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_dh, GemmFcDh, _c512, bfuse::kChunked, 512, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_dh, GemmFcDh, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512_b4, Softmax4b, gemm_gelu_f32_512x768x3072_dh, GemmFcDh, _c256, bfuse::kChunked, 256, 1)
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r3, Softmax4x3, gemm_gelu_f32_512x768x3072_dh, GemmFcDh)
BFUSE_BFUSE_RT_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_dh, GemmFcDh)
using GemmFcDh2 = GemmF32Dma<512, 3072, 768, 32, 96, 4, kEpiGeluTanh, 2>;   // two ring stages: 32 KB, so that more softmax workgroups fit beside two of these
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_dh2, GemmFcDh2, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_dh2, GemmFcDh2, _c512, bfuse::kChunked, 512, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_dh2, GemmFcDh2, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_RT_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_dh2, GemmFcDh2)
