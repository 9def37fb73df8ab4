// The dense and bgemm operators of the reference's test-utils/examples/benchmark.yaml: the layers of llm.yaml at
// 1024 rows (dense: batch, in, out) and at 1024 independent products (bgemm: batch, M, K, N), fp32, with the
// tilings of their 512-row / 16-product counterparts (model_ops.h) -- twice, or 64 times, the workgroups.
#include "fuse.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

#define DENSE_F32(M, K, N, ...)                                                                                  \
    using Dense_##M##x##K##x##N = GemmF32Dma<M, N, K, __VA_ARGS__>;                                               \
    BFUSE_KERNEL(gemm_f32_##M##x##K##x##N, Dense_##M##x##K##x##N, ({{M, K, 1, 1}, 4}), ({{K, N, 1, 1}, 4}), ({{M, N, 1, 1}, 4}))
DENSE_F32(1024, 768, 768, 32, 48, 4)
DENSE_F32(1024, 768, 3072, 32, 96, 4, kEpiNone, 2)
DENSE_F32(1024, 3072, 768, 32, 48, 4)
DENSE_F32(1024, 768, 2304, 32, 144, 4)
DENSE_F32(1024, 4096, 4096, 64, 128, 4)
DENSE_F32(1024, 4096, 1024, 32, 64, 4)
DENSE_F32(1024, 4096, 14336, 64, 128, 4)
DENSE_F32(1024, 14336, 4096, 64, 128, 4)

// C[b] = A[b] . B[b]^T, A [b, M, K], B [b, N, K]: <M, N, K, BM, BN, waves over K>
#define BGEMM_F32(B, M, K, N, BM, BN, KS)                                                                        \
    using Bgemm_##B##x##M##x##K##x##N = GemmF32<M, N, K, BM, BN, KS, kEpiNone, 2, 1, true, B>;                    \
    BFUSE_KERNEL(bgemm_f32_##B##x##M##x##K##x##N, Bgemm_##B##x##M##x##K##x##N, ({{B, M, K, 1}, 4}), ({{B, N, K, 1}, 4}), ({{B, M, N, 1}, 4}))
// the one-wave products reserve 32 KB of LDS per workgroup: four workgroups per CU, one wave per SIMD (see LdsReserve).
// (128 x 64 tiles run the K <= 128 products 7-16 % faster alone, but their 300 registers make every kernel they are part
// of a kernel of one wave per SIMD (GemmF32::MIN_WAVES_PER_EU): block-fused with them, the pairs of the reference's
// tests/interleave_scheduler suite read 0.79 of the unfused time instead of 0.90.  The operators of a fusion library
// stay good partners: 64 x 64.)
#define BGEMM_F32_RESERVE(B, M, K, N, BM, BN, KS, BYTES)                                                         \
    using Bgemm_##B##x##M##x##K##x##N = LdsReserve<GemmF32<M, N, K, BM, BN, KS, kEpiNone, 2, 1, true, B>, BYTES>; \
    BFUSE_KERNEL(bgemm_f32_##B##x##M##x##K##x##N, Bgemm_##B##x##M##x##K##x##N, ({{B, M, K, 1}, 4}), ({{B, N, K, 1}, 4}), ({{B, M, N, 1}, 4}))
BGEMM_F32_RESERVE(1024, 512, 64, 512, 64, 64, 1, 32768)
BGEMM_F32(1024, 512, 512, 64, 64, 64, 2)
BGEMM_F32_RESERVE(1024, 512, 128, 512, 64, 64, 1, 32768)
BGEMM_F32(1024, 512, 512, 128, 64, 64, 2)
BGEMM_F32_RESERVE(1024, 256, 64, 256, 64, 64, 1, 32768)
BGEMM_F32_RESERVE(1024, 256, 256, 64, 64, 64, 1, 32768)
BGEMM_F32_RESERVE(1024, 256, 80, 256, 64, 64, 1, 32768)
BGEMM_F32_RESERVE(1024, 256, 256, 80, 64, 80, 1, 32768)
BGEMM_F32_RESERVE(1024, 208, 64, 208, 112, 64, 1, 32768)
BGEMM_F32_RESERVE(1024, 208, 208, 64, 208, 32, 1, 32768)
BGEMM_F32_RESERVE(1024, 208, 80, 208, 112, 64, 1, 32768)     // 208 = 112 + 96 rows, 3 x 64 + 16 columns: the last tiles overlap their neighbours
BGEMM_F32_RESERVE(1024, 208, 208, 80, 64, 80, 1, 32768)
// tests/interleave_scheduler/config/info.yaml: bgemm_6, bgemm_7
BGEMM_F32_RESERVE(1024, 1024, 64, 512, 64, 64, 1, 32768)
BGEMM_F32(1024, 1024, 512, 64, 64, 64, 2)
