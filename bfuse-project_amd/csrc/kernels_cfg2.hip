// Pair 2 (BERT-base shapes): QKV projection GEMM [512x768].[768x2304] fp32 block-fused with
// LayerNorm over [512x768] (eps 1e-12).
#include "fuse.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// 32x144 tiles: 16 x 16 = 256 workgroups, exactly one per CU; four waves split K = 768;
// operands staged through per-wave LDS rings by direct-to-LDS loads
using GemmQkv = GemmF32Dma<512, 2304, 768, 32, 144, 4>;
// one row per one-wave workgroup (512 workgroups): the finest cut hides best behind the GEMM
using LnBert = LayerNorm<512, 768, 1, 1>;

BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, ({{512, 768, 1, 1}, 4}), ({{768, 2304, 1, 1}, 4}), ({{512, 2304, 1, 1}, 4}))
BFUSE_KERNEL(layernorm_512x768, LnBert, ({{512, 768, 1, 1}, 4}), ({{2, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))

BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, _r, bfuse::kRanges, 0, 0)
// the reference's live pattern (1:1 zig-zag) and an XCD-balanced chunking, for the record
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert, _c8, bfuse::kChunked, 8, 1)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768, LnBert)

// alternative GEMM side: operands loaded global -> VGPR directly in MFMA layout
using GemmQkvV = GemmF32<512, 2304, 768, 32, 144, 4>;
BFUSE_KERNEL(gemm_f32_512x768x2304_v, GemmQkvV, ({{512, 768, 1, 1}, 4}), ({{768, 2304, 1, 1}, 4}), ({{512, 2304, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304_v, GemmQkvV, layernorm_512x768, LnBert, _r, bfuse::kRanges, 0, 0)
// alternative LayerNorm side: four rows per four-wave workgroup (128 workgroups)
using LnBert4 = LayerNorm<512, 768, 4, 1>;
BFUSE_KERNEL(layernorm_512x768_w4, LnBert4, ({{512, 768, 1, 1}, 4}), ({{2, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x2304, GemmQkv, layernorm_512x768_w4, LnBert4, _r, bfuse::kRanges, 0, 0)
