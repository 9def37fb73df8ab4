// Pair 4 (GPT-2 small shapes, seq 512): causal softmax over 12 x [512x512] fp32 scores
// block-fused with the MLP up-projection GEMM [512x768].[768x3072] fp32 + tanh-GELU.
#include "fuse.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// softmax: one row per wave, four-wave workgroups (1536 of them)
using Softmax4 = SoftmaxCausal<12, 512, 4, 1>;
// GEMM + GELU: 16 x 32 = 512 tiles of 32 x 96, two workgroups per CU, four waves split K = 768 over
// private LDS rings of two stages (32 KB: three softmax workgroups fit beside two of these)
using GemmFc = GemmF32Dma<512, 3072, 768, 32, 96, 4, kEpiGeluTanh, 2>;

BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072, GemmFc, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))

BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072, GemmFc, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072, GemmFc, _c512, bfuse::kChunked, 512, 1)
// the reference's live pattern (1:1 zig-zag), for the record
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072, GemmFc, , bfuse::kZigzag, 1, 1)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072, GemmFc)

// alternative GEMM side: three ring stages (48 KB; 4 % faster alone, one softmax workgroup fits beside two)
using GemmFcS3 = GemmF32Dma<512, 3072, 768, 32, 96, 4, kEpiGeluTanh, 3>;
BFUSE_KERNEL(gemm_gelu_f32_512x768x3072_s3, GemmFcS3, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(softmax_causal_12x512x512, Softmax4, gemm_gelu_f32_512x768x3072_s3, GemmFcS3, _c256, bfuse::kChunked, 256, 1)
// alternative softmax side: 512 workgroups of four waves x three rows, all three rows' loads in flight;
// its grid equals the GEMM's, which is what thread-level fusion wants
using Softmax4x3 = SoftmaxCausal<12, 512, 4, 3, 3>;
BFUSE_KERNEL(softmax_causal_12x512x512_r3, Softmax4x3, ({{12, 512, 512, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_HFUSE_KERNEL(softmax_causal_12x512x512_r3, Softmax4x3, gemm_gelu_f32_512x768x3072, GemmFc)
