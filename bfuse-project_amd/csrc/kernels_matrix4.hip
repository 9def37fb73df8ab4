// The pair matrix of the reference's benchmark suite over the model operators the library holds (its
// tests/benchmark pairs every dense, bgemm and conv2d layer of its example models with every other one): each
// dense layer block-fused with each attention product and each convolution, one chunk per round over the CUs.
// Part 4 of 4 (two dense layers per file, so that the files compile side by side).
#include "fuse.h"
#include "model_ops.h"

using namespace bfuse;
using namespace bfuse::model;

BFUSE_MODULE_PROLOGUE()

BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, Dense6, bgemm_f32_12x512x64x512, Bgemm0, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, Dense6, bgemm_f32_12x512x512x64, Bgemm1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, Dense6, bgemm_f32_32x512x128x512, Bgemm2, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, Dense6, bgemm_f32_32x512x512x128, Bgemm3, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, Dense6, conv3x3_f32_64x56x56_64, Conv1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x14336, Dense6, conv3x3_f32_128x28x28_128, Conv4, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, bgemm_f32_12x512x64x512, Bgemm0, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, bgemm_f32_12x512x512x64, Bgemm1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, bgemm_f32_32x512x128x512, Bgemm2, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, bgemm_f32_32x512x512x128, Bgemm3, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, conv3x3_f32_64x56x56_64, Conv1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, conv3x3_f32_128x28x28_128, Conv4, _c256, bfuse::kChunked, 256, 1)
