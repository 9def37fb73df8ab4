// Pair 2 (BERT-base shapes): QKV projection GEMM [512x768].[768x2304] fp32 block-fused with
// LayerNorm over [512x768] (eps 1e-12).
#include "fuse.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// 32x144 tiles: 16 x 16 = 256 workgroups, exactly one per CU; four waves split K = 768
using GemmQkv = GemmF32<512, 2304, 768, 32, 144, 4>;
using LnBert = LayerNorm<512, 768, 4, 1>;

BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, ({{512, 768, 1, 1}, 4}), ({{768, 2304, 1, 1}, 4}), ({{512, 2304, 1, 1}, 4}))
BFUSE_KERNEL(layernorm_512x768, LnBert, ({{512, 768, 1, 1}, 4}), ({{2, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))

// same LayerNorm with 2 rows (256 workgroups) and 1 row (512 workgroups) per workgroup
using LnBert2 = LayerNorm<512, 768, 2, 1>;
using LnBert1 = LayerNorm<512, 768, 1, 1>;
BFUSE_KERNEL(layernorm_512x768_w2, LnBert2, ({{512, 768, 1, 1}, 4}), ({{2, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))
BFUSE_KERNEL(layernorm_512x768_w1, LnBert1, ({{512, 768, 1, 1}, 4}), ({{2, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))

BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768_w2, LnBert2, _r, bfuse::kRanges, 0, 0)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768_w1, LnBert1, _r, bfuse::kRanges, 0, 0)
BFUSE_HFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768_w2, LnBert2)

BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, _z2, bfuse::kZigzag, 2, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, _c8, bfuse::kChunked, 8, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, _r, bfuse::kRanges, 0, 0)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768_w1, LnBert1)
// operands staged through per-wave LDS rings by direct-to-LDS loads
using GemmQkvD = GemmF32Dma<512, 2304, 768, 32, 144, 4>;
BFUSE_KERNEL(gemm_f32_512x768x2304_d, GemmQkvD, ({{512, 768, 1, 1}, 4}), ({{768, 2304, 1, 1}, 4}), ({{512, 2304, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304_d, GemmQkvD, layernorm_512x768_w1, LnBert1, _r, bfuse::kRanges, 0, 0)
using GemmQkvPc = GemmF32Dma<512, 2304, 768, 32, 144, 4, kEpiNone, 3, 1>;   // + one producer wave per k-range
BFUSE_KERNEL(gemm_f32_512x768x2304_pc, GemmQkvPc, ({{512, 768, 1, 1}, 4}), ({{768, 2304, 1, 1}, 4}), ({{512, 2304, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304_pc, GemmQkvPc, layernorm_512x768_w1, LnBert1, _r, bfuse::kRanges, 0, 0)
BFUSE_BFUSE_RT_KERNEL(gemm_f32_512x768x2304_d, GemmQkvD, layernorm_512x768_w1, LnBert1)
