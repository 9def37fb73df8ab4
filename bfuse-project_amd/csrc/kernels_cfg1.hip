// Pair 1 (plumbing pair): fp32 GEMM 512x512x512 horizontally fused with y = ReLU(x + b) over
// 1 048 576 floats; 256-thread workgroups split 128 / 128 (two waves each).
#include "fuse.h"
#include "ops_gemm_f32.h"
#include "ops_rowwise.h"

using namespace bfuse;

BFUSE_MODULE_PROLOGUE()

// two waves split K; one 16x64 tile per workgroup -> 256 workgroups, one per CU
using Gemm512 = GemmF32<512, 512, 512, 16, 64, 2>;
using BiasRelu1M = BiasRelu<1048576, 128, 256>;

BFUSE_KERNEL(gemm_f32_512x512x512, Gemm512, ({{512, 512, 1, 1}, 4}), ({{512, 512, 1, 1}, 4}), ({{512, 512, 1, 1}, 4}))
BFUSE_KERNEL(bias_relu_1048576, BiasRelu1M, ({{1048576, 1, 1, 1}, 4}), ({{1048576, 1, 1, 1}, 4}), ({{1048576, 1, 1, 1}, 4}))

BFUSE_HFUSE_KERNEL(gemm_f32_512x512x512, Gemm512, bias_relu_1048576, BiasRelu1M)
BFUSE_BFUSE_KERNEL(gemm_f32_512x512x512, Gemm512, bias_relu_1048576, BiasRelu1M, , bfuse::kZigzag, 1, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x512x512, Gemm512, bias_relu_1048576, BiasRelu1M, _c8, bfuse::kChunked, 8, 1)
// the same pair with its dispatch plan as run-time data and persistent workgroups
BFUSE_BFUSE_RT_KERNEL(gemm_f32_512x512x512, Gemm512, bias_relu_1048576, BiasRelu1M)
// alternative GEMM side: four waves split K (one per SIMD); outside the configuration's 128/128 split
using Gemm512K4 = GemmF32<512, 512, 512, 16, 64, 4>;
BFUSE_KERNEL(gemm_f32_512x512x512_k4, Gemm512K4, ({{512, 512, 1, 1}, 4}), ({{512, 512, 1, 1}, 4}), ({{512, 512, 1, 1}, 4}))
BFUSE_HFUSE_KERNEL(gemm_f32_512x512x512_k4, Gemm512K4, bias_relu_1048576, BiasRelu1M)
