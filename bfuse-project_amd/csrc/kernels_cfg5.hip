// Pair 5 (Llama-3-8B shapes, seq 512): bf16 gate-projection GEMM [512x4096].[4096x14336]
// (fp32 accumulate) block-fused with RMSNorm over [512x4096] bf16 followed by RoPE on
// 32 heads x 128.
#include "fuse.h"
#include "ops_gemm_bf16.h"
#include "ops_layout.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// 128 x 224 tiles: 4 x 64 = 256 workgroups; eight compute waves (4 x 2) of 32 x 112 plus two
// producer waves that issue the direct-to-LDS loads (two, three and four producers run the same:
// 47.6-47.8 us); ring of three 64-k stages; the barrier of the next K-step before MFMA group 11 of 14
using GemmGate = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4, 4, 2, 2, 11>;
using NormRope1 = RmsNormRope<512, 32, 128, 1>;             // 512 one-wave workgroups

BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_KERNEL(rmsnorm_rope_bf16_512x4096, NormRope1, ({{512, 4096, 1, 1}, 2}), ({{(int)NormRope1::F_BYTES, 1, 1, 1}, 1}), ({{512, 4096, 1, 1}, 2}))

BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)

// Thread-level fusion: two RMSNorm+RoPE waves inside every GEMM workgroup (256 workgroups, one per
// CU, twelve waves).  The GEMM keeps the hardware barrier of its K loop; the norm waves take part
// in the first seven of them, one per section of their row (JoinSync), and leave.
using NormRope2 = RmsNormRope<512, 32, 128, 2>;             // 256 two-wave workgroups
BFUSE_KERNEL(rmsnorm_rope_bf16_512x4096_w2, NormRope2, ({{512, 4096, 1, 1}, 2}), ({{(int)NormRope2::F_BYTES, 1, 1, 1}, 1}), ({{512, 4096, 1, 1}, 2}))
BFUSE_HFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, rmsnorm_rope_bf16_512x4096_w2, NormRope2)

// alternative GEMM side: the same eight compute waves issue their own loads (no producer waves)
using GemmGate8 = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4, 4, 2>;
BFUSE_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, rmsnorm_rope_bf16_512x4096, NormRope1, _c256, bfuse::kChunked, 256, 1)
// the reference's live pattern (1:1 zig-zag), for the record, and the run-time-plan kernel (dispatch
// plan as data, persistent workgroups).  Both on the eight-wave GEMM: with ten waves the kernel is
// capped at 168 VGPRs and these two forms do not fit without spilling
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, rmsnorm_rope_bf16_512x4096, NormRope1, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_RT_KERNEL(gemm_bf16_512x4096x14336_w8, GemmGate8, rmsnorm_rope_bf16_512x4096, NormRope1)
// alternative norm side: 128 four-wave workgroups
using NormRope4 = RmsNormRope<512, 32, 128, 4>;
BFUSE_KERNEL(rmsnorm_rope_bf16_512x4096_w4, NormRope4, ({{512, 4096, 1, 1}, 2}), ({{(int)NormRope4::F_BYTES, 1, 1, 1}, 1}), ({{512, 4096, 1, 1}, 2}))
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, GemmGate, rmsnorm_rope_bf16_512x4096_w4, NormRope4, _c256, bfuse::kChunked, 256, 1)
// the headline GEMM's tiling on a K of 256: every tile position of the full 512 x 14336 output with
// dense inputs, small enough for the CPU reference to evaluate the whole matrix
using GemmGateK256 = GemmBf16NTDma<512, 14336, 256, 128, 224, 3, 4, 4, 2, 2, 11>;
BFUSE_KERNEL(gemm_bf16_512x256x14336, GemmGateK256, ({{512, 256, 1, 1}, 2}), ({{14336, 256, 1, 1}, 2}), ({{512, 14336, 1, 1}, 2}))

// a weight held as [K, N] = [4096, 14336] is brought into the GEMM's [N, K] layout once, when it is loaded
using WeightToNK = Transpose16<4096, 14336>;
BFUSE_KERNEL(transpose16_4096x14336, WeightToNK, ({{4096, 14336, 1, 1}, 2}), ({{1, 1, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}))

// The headline GEMM with clock stamps (instrumentation; `python -m bfuse_project_amd.profile_pair --clock` reads them):
// the same code with three pairs of counter reads per workgroup, its output 256 x 8 64-bit words longer.  Alone and
// with the norm waves fused in.  Not an alternative of the product kernel: its output shape differs.
using GemmGateClk = GemmBf16NTDma<512, 14336, 4096, 128, 224, 3, 4, 4, 2, 2, 11, true>;
BFUSE_KERNEL(gemm_bf16_512x4096x14336_clk, GemmGateClk, ({{512, 4096, 1, 1}, 2}), ({{14336, 4096, 1, 1}, 2}),
             ({{512 * 14336 + 256 * GemmGateClk::STAMP_WORDS * 4, 1, 1, 1}, 2}))
BFUSE_HFUSE_KERNEL(gemm_bf16_512x4096x14336_clk, GemmGateClk, rmsnorm_rope_bf16_512x4096_w2, NormRope2)
