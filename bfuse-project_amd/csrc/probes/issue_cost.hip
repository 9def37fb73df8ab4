// What does an instruction cost the wave that is streaming MFMAs?  One wave per SIMD issues 72
// independent fp32 MFMAs (16x16x4, 32 clocks each in the pipe) per iteration and, after every
// G-th of them, ONE other instruction: a vector-ALU add, an LDS read with or without address
// arithmetic, a global load to registers, a direct global->LDS load as the compiler selects it,
// or the same load with a scalar base (wave.h dma_load_lds_b128).  The clocks per MFMA over the
// pipe's 32, divided by the instructions dealt, is what one such instruction costs in MFMA issue
// time.  A last case has four extra waves per workgroup issue the loads instead.
//
//   make -C bfuse-project_amd/csrc probes && bfuse-project_amd/probe_issue_cost
#include <hip/hip_runtime.h>

#include <cstdio>

#include "../wave.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) unsigned char lds_u8;

enum Mode { kNone, kValu, kDsImm, kDsAdd, kDs64, kDs32, kGlobal, kDmaBuiltin, kDmaScalarBase, kProducer };

template <int MODE, int G>
__global__ __launch_bounds__(512, 2) void stream(const f32x4* __restrict__ src, float* out, unsigned long long* stamps, int iters)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[65536];
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
    const f32x4* p = src + (size_t)blockIdx.x * 8192 + (threadIdx.x & 255);
    const unsigned lds0 = (unsigned)(size_t)(lds_u8*)lds;
    if (MODE == kProducer && wave >= 4) {
        // a wave that only loads: twelve direct-to-LDS loads per 72 MFMAs of the wave next to it
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int l = 0; l < 12; ++l)
                bfuse::dma_load_lds_b128((unsigned)lane * 16u, reinterpret_cast<const char*>(src) + ((size_t)blockIdx.x * 8192 + (size_t)((it * 12 + l) % 48) * 1024) * 16,
                                         lds0 + (unsigned)(wave * 8 + (l & 7)) * 1024u);
            __builtin_amdgcn_s_sleep(20);
        }
        __builtin_amdgcn_s_waitcnt(0);
        return;
    }
    if (wave >= 4) return;
    f32x4 acc[2][9];
    for (int i = 0; i < 2; ++i)
        for (int c = 0; c < 9; ++c) acc[i][c] = f32x4{0, 0, 0, 0};
    float a[2][4], b[9][4];
    for (int i = 0; i < 2; ++i)
        for (int t = 0; t < 4; ++t) a[i][t] = threadIdx.x * 0.001f + i + t;
    for (int c = 0; c < 9; ++c)
        for (int t = 0; t < 4; ++t) b[c][t] = threadIdx.x * 0.002f + c - t;
    constexpr int NL = (MODE == kNone || MODE == kProducer) ? 1 : 72 / G;
    f32x4 ld[NL];
    for (int l = 0; l < NL; ++l) ld[l] = f32x4{0, 0, 0, 0};
    const unsigned long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; ++it) {
        const f32x4* q = p + (size_t)((it * 3) % 48) * 1024;
        const unsigned la = lds0 + lane * 16 + (it & 31) * 1024;
#pragma unroll
        for (int m = 0; m < 72; ++m) {
            const int t = m / 18, i = (m % 18) / 9, c = m % 9;
            acc[i][c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[i][t], b[c][t], acc[i][c], 0, 0, 0);
            if (MODE != kNone && MODE != kProducer && m % G == G - 1) {
                const int l = m / G;
                if constexpr (MODE == kValu) asm volatile("v_add_u32 %0, 1, %0" : "+v"(ld[l][0]));
                else if constexpr (MODE == kDsImm) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(ld[l]) : "v"(la), "n"((l * 1024) % 32768) : "memory");
                else if constexpr (MODE == kDsAdd) asm volatile("ds_read_b128 %0, %1" : "=v"(ld[l]) : "v"(la + (l * 1024) % 32768) : "memory");
                else if constexpr (MODE == kDs64) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(*(double*)&ld[l]) : "v"(la), "n"((l * 1024) % 32768) : "memory");
                else if constexpr (MODE == kDs32) asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(ld[l][0]) : "v"(la), "n"((l * 1024) % 32768) : "memory");
                // "+v": the destination stays allocated from one iteration to the next -- with the wait one
                // iteration late a register that looked dead could otherwise be reused (for an address,
                // say) while a load into it is still in flight
                else if constexpr (MODE == kGlobal) asm volatile("global_load_dwordx4 %0, %1, off" : "+v"(ld[l]) : "v"(q + l * 64) : "memory");
                else if constexpr (MODE == kDmaBuiltin) __builtin_amdgcn_global_load_lds(q + l * 64, (lds_u8*)lds + (wave * 8 + (l & 7)) * 1024, 16, 0, 0);
                else if constexpr (MODE == kDmaScalarBase)
                    bfuse::dma_load_lds_b128((unsigned)lane * 16u, reinterpret_cast<const char*>(src) + ((size_t)blockIdx.x * 8192 + (size_t)((it * 3) % 48) * 1024 + l * 64) * 16,
                                             lds0 + (unsigned)(wave * 8 + (l & 7)) * 1024u);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        // loads are waited for one iteration late, so that their latency is not part of the price:
        // at most this iteration's NL loads stay outstanding (vmcnt is a 6-bit count)
        if constexpr (MODE == kGlobal || MODE == kDmaScalarBase || MODE == kDmaBuiltin) __builtin_amdgcn_s_waitcnt((NL & 0xF) | ((NL >> 4) << 14) | 0x0F70);
        if constexpr (MODE == kDsImm || MODE == kDsAdd || MODE == kDs64 || MODE == kDs32) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int l = 0; l < NL; ++l) {
            asm volatile("" : "+v"(ld[l]));
            b[l % 9][l % 4] += ld[l][0] * 1e-30f;
        }
#pragma unroll
        for (int c = 0; c < 9; ++c) asm volatile("" : "+v"(b[c][0]), "+v"(b[c][1]), "+v"(b[c][2]), "+v"(b[c][3]));
    }
    const unsigned long long c1 = clock64(), w1 = wall_clock64();
    // the last iteration's loads are still in flight: their destination registers stay named until
    // they have landed (a register reused before that -- for the address of the store below, say --
    // would be overwritten by the returning data)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
    for (int l = 0; l < NL; ++l) asm volatile("" : "+v"(ld[l]));
    if (threadIdx.x == 0) {
        stamps[2 * blockIdx.x] = c1 - c0;
        stamps[2 * blockIdx.x + 1] = w1 - w0;
    }
    f32x4 s = {0, 0, 0, 0};
    for (int i = 0; i < 2; ++i)
        for (int c = 0; c < 9; ++c) s += acc[i][c];
    if (s[0] == 12345.678f) out[threadIdx.x] = s[1];   // keeps the accumulators alive; never true in practice
}

#define CHECK(call)                                                         \
    do {                                                                    \
        hipError_t e_ = (call);                                             \
        if (e_ != hipSuccess) {                                             \
            std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); \
            return 1;                                                       \
        }                                                                   \
    } while (0)

template <int MODE, int G>
int run(const char* label, const f32x4* src, float* out, unsigned long long* stamps)
{
    constexpr int kIters = 400, kGrid = 256;
    const int threads = MODE == kProducer ? 512 : 256;
    stream<MODE, G><<<kGrid, threads>>>(src, out, stamps, 50);
    CHECK(hipDeviceSynchronize());
    stream<MODE, G><<<kGrid, threads>>>(src, out, stamps, kIters);
    CHECK(hipDeviceSynchronize());
    unsigned long long h[2 * kGrid];
    CHECK(hipMemcpy(h, stamps, sizeof(h), hipMemcpyDeviceToHost));
    double cyc = 0, ref = 0;
    for (int i = 0; i < kGrid; ++i) { cyc += h[2 * i]; ref += h[2 * i + 1]; }
    cyc /= kGrid; ref /= kGrid;
    const int dealt = (MODE == kNone || MODE == kProducer) ? 0 : 72 / G;
    std::printf("%-58s %5.1f clk/MFMA  (%4.0f MHz)", label, cyc / (72.0 * kIters), cyc / (ref / 100.0));
    if (dealt) std::printf("  %5.1f clk per dealt instruction", (cyc / kIters - 72 * 32.0) / dealt);
    std::printf("\n");
    return 0;
}

int main()
{
    f32x4* src; float* out; unsigned long long* stamps;
    CHECK(hipMalloc(&src, (size_t)64 << 20));
    CHECK(hipMemset(src, 0, (size_t)64 << 20));
    CHECK(hipMalloc(&out, 4096));
    CHECK(hipMalloc(&stamps, 2 * 256 * sizeof(unsigned long long)));
    int rc = 0;
    rc |= run<kNone, 72>("MFMA only", src, out, stamps);
    rc |= run<kValu, 6>("v_add_u32 every 6 MFMAs", src, out, stamps);
    rc |= run<kDsImm, 6>("ds_read_b128, immediate offset, every 6", src, out, stamps);
    rc |= run<kDsImm, 2>("ds_read_b128, immediate offset, every 2", src, out, stamps);
    rc |= run<kDs64, 6>("ds_read_b64, immediate offset, every 6", src, out, stamps);
    rc |= run<kDs32, 6>("ds_read_b32, immediate offset, every 6", src, out, stamps);
    rc |= run<kDsAdd, 6>("ds_read_b128, address = register + v_add, every 6", src, out, stamps);
    rc |= run<kGlobal, 6>("global_load_dwordx4 (64-bit vector address), every 6", src, out, stamps);
    rc |= run<kGlobal, 12>("global_load_dwordx4 (64-bit vector address), every 12", src, out, stamps);
    rc |= run<kDmaBuiltin, 6>("global_load_lds_dwordx4 as the compiler selects it, every 6", src, out, stamps);
    rc |= run<kDmaScalarBase, 6>("global_load_lds_dwordx4, scalar base (asm), every 6", src, out, stamps);
    rc |= run<kDmaScalarBase, 12>("global_load_lds_dwordx4, scalar base (asm), every 12", src, out, stamps);
    rc |= run<kProducer, 72>("12 direct-to-LDS loads per 72 MFMAs issued by OTHER waves", src, out, stamps);
    CHECK(hipFree(src));
    CHECK(hipFree(out));
    CHECK(hipFree(stamps));
    return rc;
}
