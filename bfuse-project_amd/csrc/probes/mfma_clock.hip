// What the matrix cores of an MI355X sustain, measured instead of assumed: a dense stream of
// independent MFMAs (two waves per SIMD, 14 accumulators each, no memory traffic) on every CU,
// timed three ways at once -- HIP events (wall time), the shader clock counter and the 100 MHz
// reference counter read inside the kernel.  The ratio of the two counters is the shader
// clock the chip actually ran at; with operand values that toggle bits (random, as in a real
// GEMM) the power management holds a dense bf16 stream well below the boost clock, and that
// clock -- not the 2.4 GHz behind the published peak -- bounds any bf16 GEMM on this part.
// The bf16 stream is run with both instruction shapes (16x16x32: two A x seven B fragments;
// 32x32x16: one A x seven B), figures per 16384 flop so that they compare.
//
//   make -C bfuse-project_amd/csrc probes && bfuse-project_amd/probe_mfma_clock
#include <hip/hip_runtime.h>

#include <cstdio>
#include "../ops_ceiling.h"
// the library's own MFMA-only kernel body (the measured ceiling of the benchmark line), at this probe's length
template <bool BF16, int ITERS>
__global__ __launch_bounds__(512) void lib_stream(float* out)
{
    bfuse::NoSmem sm;
    bfuse::MfmaStream<BF16, ITERS, 1>::run((int)blockIdx.x, (int)threadIdx.x, sm, nullptr, nullptr, out, bfuse::BlockSync{});
}

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef short bf16x8 __attribute__((ext_vector_type(8)));

enum Mode { kBf16Const, kBf16Random, kF32Const, kF32Random, kBf16x32Const, kBf16x32Random };
typedef float f32x16 __attribute__((ext_vector_type(16)));

__device__ unsigned mix(unsigned x)
{
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}
// a bf16 bit pattern with random sign and mantissa and an exponent near 1.0
__device__ short random_bf16(unsigned h) { return (short)((h & 0x80ff) | 0x3c00 | ((h >> 20) & 0x300)); }

template <int MODE>
__global__ __launch_bounds__(512) void mfma_stream(float* out, unsigned long long* stamps, int iters)
{
    constexpr bool kBf16 = MODE == kBf16Const || MODE == kBf16Random;
    constexpr bool k32 = MODE == kBf16x32Const || MODE == kBf16x32Random;
    constexpr bool kRandom = MODE == kBf16Random || MODE == kF32Random || MODE == kBf16x32Random;
    f32x16 big[7];
    for (int j = 0; j < 7; ++j) for (int e = 0; e < 16; ++e) big[j][e] = 0.f;
    f32x4 acc[2][7];
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 7; ++j) acc[i][j] = f32x4{0, 0, 0, 0};
    bf16x8 a[2], b[7];
    float fa[2], fb[7];
    const unsigned t = blockIdx.x * 1024 + threadIdx.x;
    for (int i = 0; i < 2; ++i) {
        for (int e = 0; e < 8; ++e) a[i][e] = kRandom ? random_bf16(mix(t * 64 + i * 8 + e)) : (short)0x3f80;
        fa[i] = kRandom ? (float)(mix(t * 7 + i) & 0xffff) / 65536.f - 0.5f : 1.0f;
    }
    for (int j = 0; j < 7; ++j) {
        for (int e = 0; e < 8; ++e) b[j][e] = kRandom ? random_bf16(mix(t * 64 + 32 + j * 8 + e)) : (short)0x3f80;
        fb[j] = kRandom ? (float)(mix(t * 11 + j) & 0xffff) / 65536.f - 0.5f : 1.0f;
    }
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
        if constexpr (k32) {
#pragma unroll
            for (int j = 0; j < 7; ++j) big[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[0], b[j], big[j], 0, 0, 0);
        } else
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 7; ++j) {
                if constexpr (kBf16) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
                else acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
    }
    const unsigned long long c1 = clock64(), w1 = wall_clock64();
    if (threadIdx.x == 0) {
        stamps[2 * blockIdx.x] = c1 - c0;
        stamps[2 * blockIdx.x + 1] = w1 - w0;
    }
    f32x4 s = {0, 0, 0, 0};
    for (int j = 0; j < 7; ++j) s[0] += big[j][0] + big[j][15];
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 7; ++j) s += acc[i][j];
    if (s[0] == 12345.678f) out[threadIdx.x] = s[1];   // keeps the accumulators alive; never true in practice
}

#define CHECK(call)                                                                   \
    do {                                                                              \
        hipError_t e_ = (call);                                                       \
        if (e_ != hipSuccess) {                                                       \
            std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_));           \
            return 1;                                                                 \
        }                                                                             \
    } while (0)

template <bool BF16, int ITERS>
int run_lib(const char* label, float* out, double flop_per_mfma)
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 20; ++i) lib_stream<BF16, ITERS><<<256, 512>>>(out);
    CHECK(hipEventRecord(e0));
    lib_stream<BF16, ITERS><<<256, 512>>>(out);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    std::printf("%-34s %8.3f ms  %71s %7.1f TFLOP/s\n", label, ms, "", 256 * 8 * 14.0 * ITERS * flop_per_mfma / (ms * 1e-3) / 1e12);
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return 0;
}

template <int MODE>
int run(const char* label, float* out, unsigned long long* stamps, int iters, double flop_per_mfma, double pipe_clk)
{
    constexpr int kGrid = 256, kWaves = 8;
    // The chip does not give a kernel its sustained rate at once: from idle, the first 10-20 ms of a
    // dense stream run 10-25 % slower than what follows.  kWarm launches of the same length come first
    // (about 100 ms), then one launch is timed.
    constexpr int kWarm = 20;
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < kWarm; ++i) mfma_stream<MODE><<<kGrid, 64 * kWaves>>>(out, stamps, iters);
    CHECK(hipEventRecord(e0));   // no host synchronisation before the timed launch: the GPU stays busy
    mfma_stream<MODE><<<kGrid, 64 * kWaves>>>(out, stamps, iters);
    CHECK(hipEventRecord(e1));
    CHECK(hipEventSynchronize(e1));
    float ms = 0;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    unsigned long long h[2 * kGrid];
    CHECK(hipMemcpy(h, stamps, sizeof(h), hipMemcpyDeviceToHost));
    double cyc = 0, ref = 0;
    for (int i = 0; i < kGrid; ++i) { cyc += h[2 * i]; ref += h[2 * i + 1]; }
    // The SIMD issues the older wave's MFMAs first, so one wave's own loop time says little; the
    // issue interval is taken from the kernel's duration at the measured clock.
    const double mfma_per_simd = 14.0 * iters * (kWaves / 4);
    const double mhz = cyc / (ref / 100.0);
    std::printf("%-34s %8.3f ms (%.3f ms inside the kernel)  shader clock %4.0f MHz  %5.1f clk per MFMA and SIMD (pipe %2.0f)  %7.1f TFLOP/s\n", label, ms, ref / kGrid / 100.0 * 1e-3, mhz,
                ms * 1e-3 * mhz * 1e6 / mfma_per_simd, pipe_clk, kGrid * kWaves * 14.0 * iters * flop_per_mfma / (ms * 1e-3) / 1e12);
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return 0;
}

int main()
{
    float* out;
    unsigned long long* stamps;
    CHECK(hipMalloc(&out, 4 * 256 * 512));
    CHECK(hipMalloc(&stamps, 2 * 256 * sizeof(unsigned long long)));
    int rc = 0;
    for (int rep = 0; rep < 2 && !rc; ++rep) {
        rc |= run<kBf16Const>("bf16 16x16x32, constant operands", out, stamps, 20000, 16384.0, 16);
        rc |= run<kBf16Random>("bf16 16x16x32, random operands", out, stamps, 20000, 16384.0, 16);
        rc |= run<kBf16x32Const>("bf16 32x32x16, constant operands", out, stamps, 20000, 16384.0, 16);
        rc |= run<kBf16x32Random>("bf16 32x32x16, random operands", out, stamps, 20000, 16384.0, 16);
        rc |= run<kF32Const>("f32 16x16x4, constant operands", out, stamps, 10000, 2048.0, 32);
        rc |= run<kF32Random>("f32 16x16x4, random operands", out, stamps, 10000, 2048.0, 32);
        rc |= run_lib<true, 20000>("library body, bf16 16x16x32, random", out, 16384.0);
        rc |= run_lib<false, 10000>("library body, f32 16x16x4, random", out, 2048.0);
    }
    CHECK(hipFree(out));
    CHECK(hipFree(stamps));
    return rc;
}
