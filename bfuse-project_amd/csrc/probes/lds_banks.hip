// Which lane -> address patterns of an LDS access are free of bank conflicts on gfx950?  Four waves
// (one per SIMD) of one workgroup repeat ONE LDS instruction whose per-lane byte address comes from
// a host-built table; clocks per instruction per wave tell how many passes the LDS needed.  The
// patterns are the ones the kernels of this library use or rejected: MFMA fragment reads out of
// row-major tiles of several pitches, the convolution's tap reads and staging stores.
//
//   make -C bfuse-project_amd/csrc probes && bfuse-project_amd/probe_lds_banks
#include <hip/hip_runtime.h>

#include <cstdio>
#include <functional>
#include <vector>

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) unsigned char lds_u8;

enum Op { kR32, kR64, kR128, kW32, kW64, kW128 };

template <int OP>
__global__ __launch_bounds__(1024) void hammer(const unsigned* __restrict__ offs, unsigned long long* stamps, float* out, int iters)
{
    __shared__ __attribute__((aligned(1024))) unsigned char lds[65536];
    const int lane = threadIdx.x & 63;
    for (int i = threadIdx.x; i < 65536 / 4; i += blockDim.x) reinterpret_cast<float*>(lds)[i] = 0.f;
    __syncthreads();
    const unsigned a = (unsigned)(size_t)(lds_u8*)lds + offs[lane];
    f32x4 v[8];
    for (int i = 0; i < 8; ++i) v[i] = f32x4{1.f * lane, 2.f, 3.f, 4.f};
    const unsigned long long c0 = clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            if constexpr (OP == kR32) asm volatile("ds_read_b32 %0, %1" : "=v"(v[i][0]) : "v"(a) : "memory");
            else if constexpr (OP == kR64) asm volatile("ds_read_b64 %0, %1" : "=v"(*(f32x2*)&v[i]) : "v"(a) : "memory");
            else if constexpr (OP == kR128) asm volatile("ds_read_b128 %0, %1" : "=v"(v[i]) : "v"(a) : "memory");
            else if constexpr (OP == kW32) asm volatile("ds_write_b32 %0, %1" : : "v"(a), "v"(v[i][0]) : "memory");
            else if constexpr (OP == kW64) asm volatile("ds_write_b64 %0, %1" : : "v"(a), "v"(*(f32x2*)&v[i]) : "memory");
            else asm volatile("ds_write_b128 %0, %1" : : "v"(a), "v"(v[i]) : "memory");
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(v[i]));
    }
    const unsigned long long c1 = clock64();
    if (lane == 0) stamps[threadIdx.x >> 6] = c1 - c0;
    float s = 0;
    for (int i = 0; i < 8; ++i) s += v[i][0] + v[i][3];
    if (s == 12345.678f) out[threadIdx.x] = s;
}

#define CHECK(call)                                                         \
    do {                                                                    \
        hipError_t e_ = (call);                                             \
        if (e_ != hipSuccess) {                                             \
            std::fprintf(stderr, "%s: %s\n", #call, hipGetErrorString(e_)); \
            return 1;                                                       \
        }                                                                   \
    } while (0)

static unsigned* d_offs; static unsigned long long* d_stamps; static float* d_out;

template <int OP>
int run(const char* label, int width, const std::function<unsigned(int)>& f, int waves = 4)
{
    unsigned h[64];
    for (int l = 0; l < 64; ++l) {
        h[l] = f(l);
        if (h[l] % width || h[l] + width > 65536) { std::fprintf(stderr, "%s: bad offset %u for lane %d\n", label, h[l], l); return 1; }
    }
    CHECK(hipMemcpy(d_offs, h, sizeof(h), hipMemcpyHostToDevice));
    constexpr int kIters = 2000;
    hammer<OP><<<1, 64 * waves>>>(d_offs, d_stamps, d_out, 200);
    CHECK(hipDeviceSynchronize());
    hammer<OP><<<1, 64 * waves>>>(d_offs, d_stamps, d_out, kIters);
    CHECK(hipDeviceSynchronize());
    unsigned long long s[16];
    CHECK(hipMemcpy(s, d_stamps, sizeof(unsigned long long) * waves, hipMemcpyDeviceToHost));
    double m = 0;
    for (int i = 0; i < waves; ++i) m = s[i] > m ? (double)s[i] : m;
    // the waves share the LDS: clocks per instruction of the CU's LDS
    std::printf("%-74s %6.2f clk / wave instruction\n", label, m / (kIters * 8.0 * waves));
    return 0;
}

int main()
{
    CHECK(hipMalloc(&d_offs, 256));
    CHECK(hipMalloc(&d_stamps, 256));
    CHECK(hipMalloc(&d_out, 4096));
    int rc = 0;
    auto li = [](int l) { return l & 15; };
    auto kq = [](int l) { return l >> 4; };
    // ---- 128-bit reads
    rc |= run<kR128>("b128 read   contiguous: lane*16", 16, [&](int l) { return l * 16u; });
    rc |= run<kR128>("b128 read   contiguous, 8 waves", 16, [&](int l) { return l * 16u; }, 8);
    rc |= run<kR128>("b128 read   contiguous, 12 waves", 16, [&](int l) { return l * 16u; }, 12);
    rc |= run<kR128>("b128 read   all lanes one address", 16, [&](int l) { return 0u; });
    rc |= run<kR128>("b128 read   lane*32 (every other slot)", 16, [&](int l) { return l * 32u; });
    for (unsigned pitch : {1024u, 1152u, 1536u, 1024u + 16, 1024u + 32, 1024u + 64, 1024u + 128})
    {
        char name[128];
        std::snprintf(name, sizeof name, "b128 read   kq*%u + li*16   (pitch = %u mod 256)", pitch, pitch % 256);
        rc |= run<kR128>(name, 16, [&](int l) { return kq(l) * pitch + li(l) * 16u; });
    }
    rc |= run<kR128>("b128 read   conv tap with a row wrap: kq*PLANE + (li + 2*(li>=9))*16", 16, [&](int l) { return kq(l) * 3088u + (li(l) + 2 * (li(l) >= 9)) * 16u; });
    // bf16 MFMA fragment out of a [rows][64 k] tile (128-byte rows, 8 chunks of 16 bytes): lane (li, kq) reads chunk kq of row li
    rc |= run<kR128>("b128 read   bf16 fragment, rows of 128 B: li*128 + kq*16", 16, [&](int l) { return li(l) * 128u + kq(l) * 16u; });
    rc |= run<kR128>("b128 read   bf16 fragment, chunk c of row r at c ^ ((r >> 1) & 7)", 16, [&](int l) { return li(l) * 128u + ((kq(l) ^ ((li(l) >> 1) & 7))) * 16u; });
    rc |= run<kR128>("b128 read   bf16 fragment, chunk c of row r at c ^ (r & 7)", 16, [&](int l) { return li(l) * 128u + ((kq(l) ^ (li(l) & 7))) * 16u; });
    // ---- 64-bit reads
    rc |= run<kR64>("b64 read    contiguous: lane*8", 8, [&](int l) { return l * 8u; });
    rc |= run<kR64>("b64 read    A fragment: li*32 + kq*8", 8, [&](int l) { return li(l) * 32u + kq(l) * 8u; });
    rc |= run<kR64>("b64 read    A fragment, halves swapped for rows >= 8", 8, [&](int l) { return li(l) * 32u + (((kq(l) >> 1) ^ (li(l) >> 3)) & 1) * 16u + (kq(l) & 1) * 8u; });
    rc |= run<kR64>("b64 read    A fragment, [half][row][16 B]", 8, [&](int l) { return (kq(l) >> 1) * 256u + li(l) * 16u + (kq(l) & 1) * 8u; });
    rc |= run<kR64>("b64 read    lane*16", 8, [&](int l) { return l * 16u; });
    // ---- 32-bit reads
    rc |= run<kR32>("b32 read    contiguous: lane*4", 4, [&](int l) { return l * 4u; });
    rc |= run<kR32>("b32 read    B fragment: (2kq*144 + li)*4", 4, [&](int l) { return (2 * kq(l) * 144u + li(l)) * 4u; });
    rc |= run<kR32>("b32 read    B fragment: (2kq*(144+8) + li)*4", 4, [&](int l) { return (2 * kq(l) * 152u + li(l)) * 4u; });
    rc |= run<kR32>("b32 read    lane*8", 4, [&](int l) { return l * 8u; });
    // ---- writes
    rc |= run<kW32>("b32 write   contiguous: lane*4", 4, [&](int l) { return l * 4u; });
    rc |= run<kW32>("b32 write   conv staging: (cl/4)*PLANE + c4*64 + (cl%4)*4, cl = lane/4", 4, [&](int l) { int cl = l >> 2, c4 = l & 3; return (cl / 4) * 3088u + c4 * 64u + (cl % 4) * 4u; });
    rc |= run<kW32>("b32 write   conv staging, chunk index fastest: cl = lane%16", 4, [&](int l) { int cl = l & 15, c4 = l >> 4; return (cl / 4) * 3072u + c4 * 64u + (cl % 4) * 4u; });
    rc |= run<kW64>("b64 write   contiguous: lane*8", 8, [&](int l) { return l * 8u; });
    rc |= run<kW128>("b128 write  contiguous: lane*16", 16, [&](int l) { return l * 16u; });
    rc |= run<kW128>("b128 write  contiguous, 8 waves", 16, [&](int l) { return l * 16u; }, 8);
    rc |= run<kW128>("b128 write  lane*32", 16, [&](int l) { return l * 32u; });
    return rc;
}
