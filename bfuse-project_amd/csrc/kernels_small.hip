// Small instances of every operator body and fusion form.  They exist for the parity tests:
// shapes the CPU oracle evaluates in full, tile configurations the five headline pairs do
// not reach (single-wave GEMM without LDS reduction, 16-column groups only, deeper
// prefetch, multi-group convolution, several K-steps / M-tiles of the bf16 GEMM), sides with
// different grid sizes under horizontal fusion, and the ratio / proportional block patterns.
#include "fuse.h"
#include "ops_ceiling.h"
#include "ops_conv.h"
#include "ops_conv_1x1.h"
#include "ops_gemm_bf16.h"
#include "ops_gemm_f32.h"
#include "ops_gemm_f32_dma.h"
#include "ops_layout.h"
#include "ops_pool.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// Test operator for the side barrier's give-up path: the two waves of a workgroup swap their
// values through LDS across one barrier, y[g] = x[partner of g] + f[g].  Under a side barrier
// (GroupSync) wave 0 then takes ONE MORE barrier that wave 1 never reaches: the wait is bounded, so
// it gives up, the kernel ends normally with the right output, and the host must report
// BFUSE_ERR_SYNC.  Under the hardware barrier (standalone, block fusion) the body is well formed.
template <int NBLOCKS_, int TAG_>
struct SyncProbe {
    static constexpr int THREADS = 128;
    static constexpr Dims3 GRID{NBLOCKS_, 1, 1};
    static constexpr Dims3 BLOCK{THREADS, 1, 1};
    static constexpr bool HAS_BARRIERS = true;
    struct Smem {
        float v[THREADS];
    };
    template <class Sync>
    __device__ static __forceinline__ void run(int vblock, int tid, Smem& sm, const void* I, const void* F, void* O, Sync sync)
    {
        const int g = vblock * THREADS + tid;
        sm.v[tid] = static_cast<const float*>(I)[g];
        sync();
        static_cast<float*>(O)[g] = sm.v[tid ^ 64] + static_cast<const float*>(F)[g];
        if constexpr (std::is_same<Sync, GroupSync>::value) {
            if (tid < 64) sync();   // unmatched on purpose: bounded wait, then the give-up is recorded
        }
    }
};
using SyncProbeA = SyncProbe<4, 0>;
using SyncProbeB = SyncProbe<6, 1>;

using GemmS1 = GemmF32<64, 48, 32, 16, 48, 1>;                        // one wave, a 32- and a 16-column group
using GemmS2 = GemmF32<96, 192, 128, 32, 64, 2, kEpiGeluTanh, 3>;     // 2 waves, GELU, 3 register stages
using GemmS3 = GemmF32<32, 144, 256, 32, 144, 4>;                     // the 64+64+16 column split, one tile
using GemmS7 = GemmF32<80, 112, 32, 32, 64, 1>;                        // tiles that do not divide the problem: rows 0, 32, 48 and columns 0, 48 (the last tiles overlap their neighbours)
using GemmS8 = GemmF32<48, 80, 64, 32, 64, 2, kEpiNone, 2, 1, true, 3>;   // the same on three batched products with B [N, K] and two waves over K
using GemmS9 = GemmF32<256, 64, 32, 128, 64, 1>;                       // 128 x 64 tiles: 32 accumulator blocks, a kernel of one wave per SIMD (MIN_WAVES_PER_EU), also when fused
using GemmS5 = GemmF32Dma<128, 192, 160, 32, 96, 2>;                  // private LDS rings, two waves split K, ten 8-k stages each
using GemmS6 = GemmF32Dma<64, 288, 192, 32, 144, 4, kEpiGeluTanh>;    // the 32x144 tile (partial last B load), four waves, GELU
using BiasReluS = BiasRelu<4096, 64, 4>;
using LayerNormS = LayerNorm<8, 256, 2, 1>;
using SoftmaxS = SoftmaxCausal<2, 256, 2, 2, 2>;
using ConvS1 = Conv3x3F32Lds<16, 16, 8, 8, 16, 1, 1>;                 // one channel group, one wave
using ConvS2 = Conv3x3F32Lds<32, 32, 12, 12, 16, 1, 2>;               // two channel groups on two waves
using ConvS3 = Conv3x3F32Lds<64, 16, 8, 16, 16, 2, 2>;                // two groups per wave, two pixel blocks
using PoolS = MaxPool3x3S2<4, 16, 16, 64>;
using Conv1S1 = Conv1x1F32<32, 32, 5, 5, 1, 32, 4, 3>;                 // streamed 1x1: three images of 25 pixels = three ragged tiles in one workgroup, its fourth wave without a tile
using Conv1S2 = Conv1x1F32<96, 48, 9, 9, 1, 16, 2, 5>;                 // 64 + 17 pixels per image, three channel tiles, two filter chunks of 48 channels (192 staging units on 128 threads)
using Conv1S3 = Conv1x1F32<16, 16, 9, 7, 2, 16, 1, 2>;                 // stride 2 (9 x 7 -> 5 x 4), one wave per workgroup: no barrier
using GemmB1 = GemmBf16NTDma<128, 1792, 64, 128, 224, 2>;             // one K-step
using GemmB2 = GemmBf16NTDma<128, 1792, 192, 128, 224, 2>;            // two stages, three K-steps
using GemmB3 = GemmBf16NTDma<256, 1792, 320, 128, 224, 3>;            // two M-tiles, ring of three, five K-steps
using GemmB5 = GemmBf16NTDma<256, 1792, 320, 128, 224, 3, 4, 4, 2>;   // the same with eight waves (uneven load groups per wave)
using GemmB8 = GemmBf16NTDma<256, 1792, 384, 128, 224, 3, 4, 4, 2, 4, 11>;   // eight compute + four producer waves, early barrier, six K-steps (all after the rolled loop)
using GemmB9 = GemmBf16NTDma<256, 1792, 448, 128, 224, 3, 4, 4, 2, 2, 10>;   // eight compute + two producer waves, early barrier, seven K-steps (one round of the rolled loop, then the last step)
using GemmB11 = GemmBf16NTDma<128, 1024, 320, 64, 128, 3, 2, 2, 2, 2, 6>;   // 64 x 128 tiles, four compute waves (2 x 2) of 32 x 64 + two producer waves, read-ahead of two, early barrier
using NormRopeS = RmsNormRope<6, 8, 128, 2>;

BFUSE_KERNEL(gemm_f32_64x32x48, GemmS1, ({{64, 32, 1, 1}, 4}), ({{32, 48, 1, 1}, 4}), ({{64, 48, 1, 1}, 4}))
BFUSE_KERNEL(gemm_gelu_f32_96x128x192, GemmS2, ({{96, 128, 1, 1}, 4}), ({{128, 192, 1, 1}, 4}), ({{96, 192, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_32x256x144, GemmS3, ({{32, 256, 1, 1}, 4}), ({{256, 144, 1, 1}, 4}), ({{32, 144, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_80x32x112, GemmS7, ({{80, 32, 1, 1}, 4}), ({{32, 112, 1, 1}, 4}), ({{80, 112, 1, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_3x48x64x80, GemmS8, ({{3, 48, 64, 1}, 4}), ({{3, 80, 64, 1}, 4}), ({{3, 48, 80, 1}, 4}))
BFUSE_KERNEL(gemm_f32_256x32x64_t128, GemmS9, ({{256, 32, 1, 1}, 4}), ({{32, 64, 1, 1}, 4}), ({{256, 64, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_128x160x192_d, GemmS5, ({{128, 160, 1, 1}, 4}), ({{160, 192, 1, 1}, 4}), ({{128, 192, 1, 1}, 4}))
BFUSE_KERNEL(gemm_gelu_f32_64x192x288_d, GemmS6, ({{64, 192, 1, 1}, 4}), ({{192, 288, 1, 1}, 4}), ({{64, 288, 1, 1}, 4}))
BFUSE_KERNEL(bias_relu_4096, BiasReluS, ({{4096, 1, 1, 1}, 4}), ({{4096, 1, 1, 1}, 4}), ({{4096, 1, 1, 1}, 4}))
BFUSE_KERNEL(layernorm_8x256, LayerNormS, ({{8, 256, 1, 1}, 4}), ({{2, 256, 1, 1}, 4}), ({{8, 256, 1, 1}, 4}))
BFUSE_KERNEL(softmax_causal_2x256x256, SoftmaxS, ({{2, 256, 256, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{2, 256, 256, 1}, 4}))
BFUSE_KERNEL(conv3x3_f32_16x8x8_16, ConvS1, ({{1, 16, 8, 8}, 4}), ({{16, 16, 3, 3}, 4}), ({{1, 16, 8, 8}, 4}))
BFUSE_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, ({{1, 32, 12, 12}, 4}), ({{32, 32, 3, 3}, 4}), ({{1, 32, 12, 12}, 4}))
BFUSE_KERNEL(conv3x3_f32_64x8x16_16, ConvS3, ({{1, 64, 8, 16}, 4}), ({{16, 64, 3, 3}, 4}), ({{1, 16, 8, 16}, 4}))
BFUSE_KERNEL(conv1x1s1p0_f32_3x32x5x5_32, Conv1S1, ({{3, 32, 5, 5}, 4}), ({{32, 32, 1, 1}, 4}), ({{3, 32, 5, 5}, 4}))
BFUSE_KERNEL(conv1x1s1p0_f32_5x96x9x9_48, Conv1S2, ({{5, 96, 9, 9}, 4}), ({{48, 96, 1, 1}, 4}), ({{5, 48, 9, 9}, 4}))
BFUSE_KERNEL(conv1x1s2p0_f32_2x16x9x7_16, Conv1S3, ({{2, 16, 9, 7}, 4}), ({{16, 16, 1, 1}, 4}), ({{2, 16, 5, 4}, 4}))
BFUSE_KERNEL(maxpool3x3s2_f32_4x16x16, PoolS, ({{1, 4, 16, 16}, 4}), ({{1, 1, 1, 1}, 4}), ({{1, 4, 8, 8}, 4}))
BFUSE_KERNEL(gemm_bf16_128x64x1792, GemmB1, ({{128, 64, 1, 1}, 2}), ({{1792, 64, 1, 1}, 2}), ({{128, 1792, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_128x192x1792, GemmB2, ({{128, 192, 1, 1}, 2}), ({{1792, 192, 1, 1}, 2}), ({{128, 1792, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_256x320x1792, GemmB3, ({{256, 320, 1, 1}, 2}), ({{1792, 320, 1, 1}, 2}), ({{256, 1792, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_256x320x1792_w8, GemmB5, ({{256, 320, 1, 1}, 2}), ({{1792, 320, 1, 1}, 2}), ({{256, 1792, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_256x384x1792_p, GemmB8, ({{256, 384, 1, 1}, 2}), ({{1792, 384, 1, 1}, 2}), ({{256, 1792, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_256x448x1792_p2, GemmB9, ({{256, 448, 1, 1}, 2}), ({{1792, 448, 1, 1}, 2}), ({{256, 1792, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_128x320x1024_t64, GemmB11, ({{128, 320, 1, 1}, 2}), ({{1024, 320, 1, 1}, 2}), ({{128, 1024, 1, 1}, 2}))
BFUSE_KERNEL(rmsnorm_rope_bf16_6x1024, NormRopeS, ({{6, 1024, 1, 1}, 2}), ({{(int)NormRopeS::F_BYTES, 1, 1, 1}, 1}), ({{6, 1024, 1, 1}, 2}))

// [128, 192] -> [192, 128], 16-bit elements: 2 x 3 tiles
using TransposeS = Transpose16<128, 192>;
BFUSE_KERNEL(transpose16_128x192, TransposeS, ({{128, 192, 1, 1}, 2}), ({{1, 1, 1, 1}, 2}), ({{192, 128, 1, 1}, 2}))

// calibration kernel for the memory counters: 64 MiB read, 64 MiB written
using Copy64M = CopyF32<16777216, 256>;
BFUSE_KERNEL(copy_f32_16777216, Copy64M, ({{16777216, 1, 1, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{16777216, 1, 1, 1}, 4}))

// what the matrix cores sustain with nothing else going on: 2000 (bf16) / 1000 (fp32) rounds of 14
// independent MFMAs per wave, 0.94 TFLOP / 0.059 TFLOP per launch (about 0.6 / 0.4 ms)
using MfmaStreamBf16 = MfmaStream<true, 2000>;
using MfmaStreamF32 = MfmaStream<false, 1000>;
BFUSE_KERNEL(mfma_stream_bf16_2000, MfmaStreamBf16, ({{1, 1, 1, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{256, 512, 1, 1}, 4}))
BFUSE_KERNEL(mfma_stream_f32_1000, MfmaStreamF32, ({{1, 1, 1, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{256, 512, 1, 1}, 4}))

// horizontal fusion with unequal grids (9 GEMM tiles, 4 element-wise blocks) and a barrier side
BFUSE_HFUSE_KERNEL(gemm_gelu_f32_96x128x192, GemmS2, bias_relu_4096, BiasReluS)
// both sides carry a barrier: two LDS-counter barriers in one workgroup
BFUSE_HFUSE_KERNEL(gemm_gelu_f32_96x128x192, GemmS2, conv3x3_f32_32x12x12_32, ConvS2)
// ratio 2:1 zig-zag (18 conv tiles, 9 GEMM tiles), proportional, chunked with a remainder
BFUSE_BFUSE_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, , bfuse::kZigzag, 2, 1)
BFUSE_BFUSE_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, _p1, bfuse::kProportional, 1, 1)
BFUSE_BFUSE_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2, _c4, bfuse::kChunked, 4, 1)
BFUSE_BFUSE_KERNEL(layernorm_8x256, LayerNormS, softmax_causal_2x256x256, SoftmaxS, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_256x320x1792, GemmB3, rmsnorm_rope_bf16_6x1024, NormRopeS, _c8, bfuse::kChunked, 8, 1)
BFUSE_HFUSE_KERNEL(maxpool3x3s2_f32_4x16x16, PoolS, layernorm_8x256, LayerNormS)
// a side with a barrier in its K loop under horizontal fusion, both sides synchronising: its fence-free
// barriers become the LDS-counter one
BFUSE_HFUSE_KERNEL(gemm_bf16_256x320x1792_w8, GemmB5, gemm_f32_128x160x192_d, GemmS5)
// (the producer-wave GEMMs are not paired with a synchronising partner: their K loop under the LDS-counter
// barrier needs more scalar registers than there are, and the build refuses kernels that spill)
// the same GEMM with producer waves keeps the hardware barrier in its K loop and the norm waves join
// its first four barriers (16 GEMM tiles, 3 norm workgroups: most workgroups have no norm waves at all)
BFUSE_HFUSE_KERNEL(gemm_bf16_256x384x1792_p, GemmB8, rmsnorm_rope_bf16_6x1024, NormRopeS)
BFUSE_HFUSE_KERNEL(gemm_bf16_256x448x1792_p2, GemmB9, rmsnorm_rope_bf16_6x1024, NormRopeS)
// run-time plans / persistent workgroups: equal and unequal workgroup widths, barrier-bearing sides
BFUSE_BFUSE_RT_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, gemm_gelu_f32_96x128x192, GemmS2)
BFUSE_BFUSE_RT_KERNEL(layernorm_8x256, LayerNormS, softmax_causal_2x256x256, SoftmaxS)
BFUSE_BFUSE_RT_KERNEL(gemm_bf16_256x320x1792_w8, GemmB5, rmsnorm_rope_bf16_6x1024, NormRopeS)
BFUSE_BFUSE_RT_KERNEL(gemm_f32_128x160x192_d, GemmS5, bias_relu_4096, BiasReluS)
BFUSE_HFUSE_KERNEL(gemm_f32_128x160x192_d, GemmS5, bias_relu_4096, BiasReluS)
BFUSE_BFUSE_KERNEL(gemm_gelu_f32_64x192x288_d, GemmS6, layernorm_8x256, LayerNormS, _c4, bfuse::kChunked, 4, 1)
BFUSE_HFUSE_KERNEL(conv3x3_f32_32x12x12_32, ConvS2, bias_relu_4096, BiasReluS)
BFUSE_BFUSE_KERNEL(conv3x3_f32_64x8x16_16, ConvS3, layernorm_8x256, LayerNormS, _c4, bfuse::kChunked, 4, 1)
// both sides synchronise (each split-K GEMM's reduction barriers): each side gets LDS arrival counters of its own
BFUSE_HFUSE_KERNEL(gemm_f32_128x160x192_d, GemmS5, gemm_gelu_f32_64x192x288_d, GemmS6)
// the streamed 1x1 convolution (a barrier per filter chunk): block-fused, thread-fused with a side that never
// synchronises, and with one that does
BFUSE_BFUSE_KERNEL(conv1x1s1p0_f32_3x32x5x5_32, Conv1S1, layernorm_8x256, LayerNormS, _c4, bfuse::kChunked, 4, 1)
BFUSE_HFUSE_KERNEL(conv1x1s1p0_f32_5x96x9x9_48, Conv1S2, bias_relu_4096, BiasReluS)
BFUSE_HFUSE_KERNEL(conv1x1s1p0_f32_5x96x9x9_48, Conv1S2, conv3x3_f32_32x12x12_32, ConvS2)
BFUSE_BFUSE_KERNEL(conv1x1s2p0_f32_2x16x9x7_16, Conv1S3, bias_relu_4096, BiasReluS, , bfuse::kZigzag, 1, 1)
// a side that needs more than the 256 registers of two waves per SIMD: the fused kernels are compiled for one
static_assert(bfuse::min_waves<GemmS9>() == 1 && bfuse::min_waves<GemmS9, BiasReluS>() == 1 && bfuse::min_waves<GemmS1, BiasReluS>() == bfuse::kMinWavesPerEu,
              "a fused kernel takes the smallest wave count of its sides");
BFUSE_BFUSE_KERNEL(gemm_f32_256x32x64_t128, GemmS9, bias_relu_4096, BiasReluS, , bfuse::kZigzag, 1, 1)
BFUSE_HFUSE_KERNEL(gemm_f32_256x32x64_t128, GemmS9, bias_relu_4096, BiasReluS)
// overlapping last tiles: the shared elements are written twice with the same bits, also inside fused kernels
BFUSE_BFUSE_KERNEL(gemm_f32_80x32x112, GemmS7, layernorm_8x256, LayerNormS, , bfuse::kZigzag, 1, 1)
BFUSE_HFUSE_KERNEL(bgemm_f32_3x48x64x80, GemmS8, bias_relu_4096, BiasReluS)
// the give-up path of the side barrier, forced from the host with a small spin limit
BFUSE_KERNEL(selftest_sync_a, SyncProbeA, ({{512, 1, 1, 1}, 4}), ({{512, 1, 1, 1}, 4}), ({{512, 1, 1, 1}, 4}))
BFUSE_KERNEL(selftest_sync_b, SyncProbeB, ({{768, 1, 1, 1}, 4}), ({{768, 1, 1, 1}, 4}), ({{768, 1, 1, 1}, 4}))
BFUSE_HFUSE_KERNEL(selftest_sync_a, SyncProbeA, selftest_sync_b, SyncProbeB)
