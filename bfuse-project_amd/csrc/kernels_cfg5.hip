// Pair 5 (Llama-3-8B shapes, seq 512): bf16 gate-projection GEMM [512x4096].[4096x14336]
// (fp32 accumulate) block-fused with RMSNorm over [512x4096] bf16 followed by RoPE on
// 32 heads x 128.
#include "fuse.h"
#include "ops_gemm_bf16.h"
#include "ops_gemm_bf16_ring.h"
#include "ops_gemm_bf16_x32.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

using GemmGate = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4>;   // 4 x 64 = 256 workgroups, direct-to-LDS ring
using GemmGate8 = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4, 4, 2>;   // same tiles, eight waves of 32 x 112 (two per SIMD)
using GemmGateP = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4, 4, 2, 4>;   // eight compute waves + four producer waves that issue the loads
using GemmGateX = GemmBf16NT32<512, 14336, 4096, 128, 224, 3, 3, 4>;   // 32x32x16 MFMAs: waves of 32 x 128 and 32 x 96, four producer waves
using GemmGateR = GemmBf16NTRing<512, 14336, 4096, 128, 224, 7, 4, 2>;     // 32-k stages in a ring of seven, barrier inside the stage, continuous MFMA stream
using GemmGateV = GemmBf16NT<512, 14336, 4096, 128, 224>;           // same tiles, operands staged through VGPRs
using NormRope1 = RmsNormRope<512, 32, 128, 1>;             // 512 one-wave workgroups
using NormRope4 = RmsNormRope<512, 32, 128, 4>;             // 128 four-wave workgroups

BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x4096x14336_p, GemmGateP, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x4096x14336_x, GemmGateX, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x4096x14336_r, GemmGateR, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x4096x14336_v, GemmGateV, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(rmsnorm_rope_bf16_512x4096, NormRope1, ({{512, 4096, 1, 1}, 2}), ({{(int)NormRope1::F_BYTES, 1, 1, 1}, 1}), ({{512, 4096, 1, 1}, 2}))
BFUSE_KERNEL(rmsnorm_rope_bf16_512x4096_w4, NormRope4, ({{512, 4096, 1, 1}, 2}), ({{(int)NormRope4::F_BYTES, 1, 1, 1}, 1}), ({{512, 4096, 1, 1}, 2}))

BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, rmsnorm_rope_bf16_512x4096, NormRope1, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, rmsnorm_rope_bf16_512x4096_w4, NormRope4, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_v, GemmGateV, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_r, GemmGateR, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, rmsnorm_rope_bf16_512x4096, NormRope1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_p, GemmGateP, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_x, GemmGateX, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
