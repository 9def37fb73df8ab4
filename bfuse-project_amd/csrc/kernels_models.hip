// Further layers of the reference's example models (test-utils/examples/llm.yaml, resnet-18.yaml), beyond the
// ones the five benchmark configurations use: the same templates at other shapes (model_ops.h), so that the ids
// of those files resolve to kernels of the library (bfuse_project_amd.configure).
#include "fuse.h"
#include "model_ops.h"

using namespace bfuse;
using namespace bfuse::model;

BFUSE_MODULE_PROLOGUE()

BFUSE_KERNEL(gemm_f32_512x768x768, Dense0, ({{512, 768, 1, 1}, 4}), ({{768, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_512x768x3072, Dense1, ({{512, 768, 1, 1}, 4}), ({{768, 3072, 1, 1}, 4}), ({{512, 3072, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_512x3072x768, Dense2, ({{512, 3072, 1, 1}, 4}), ({{3072, 768, 1, 1}, 4}), ({{512, 768, 1, 1}, 4}))
BFUSE_KERNEL(gemm_f32_512x4096x1024, Dense5, ({{512, 4096, 1, 1}, 4}), ({{4096, 1024, 1, 1}, 4}), ({{512, 1024, 1, 1}, 4}))
BFUSE_KERNEL(gemm_bf16_512x4096x4096, Dense4, ({{512, 4096, 1, 1}, 2}), ({{4096, 4096, 1, 1}, 2}), ({{512, 4096, 1, 1}, 2}))
BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, ({{512, 14336, 1, 1}, 2}), ({{4096, 14336, 1, 1}, 2}), ({{512, 4096, 1, 1}, 2}))
BFUSE_KERNEL(conv3x3_f32_128x28x28_128, Conv4, ({{1, 128, 28, 28}, 4}), ({{128, 128, 3, 3}, 4}), ({{1, 128, 28, 28}, 4}))
BFUSE_KERNEL(bgemm_f32_12x512x64x512, Bgemm0, ({{12, 512, 64, 1}, 4}), ({{12, 512, 64, 1}, 4}), ({{12, 512, 512, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_12x512x512x64, Bgemm1, ({{12, 512, 512, 1}, 4}), ({{12, 64, 512, 1}, 4}), ({{12, 512, 64, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_32x512x128x512, Bgemm2, ({{32, 512, 128, 1}, 4}), ({{32, 512, 128, 1}, 4}), ({{32, 512, 512, 1}, 4}))
BFUSE_KERNEL(bgemm_f32_32x512x512x128, Bgemm3, ({{32, 512, 512, 1}, 4}), ({{32, 128, 512, 1}, 4}), ({{32, 512, 128, 1}, 4}))

// each with a memory-bound partner, block-fused one chunk per round over the CUs: the LayerNorm of pair 2 for the
// fp32 layers, RMSNorm + RoPE of pair 5 for the bf16 ones, the causal softmax that follows it in the model for the
// attention scores
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x768, Dense0, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x768x3072, Dense1, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x3072x768, Dense2, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_f32_512x4096x1024, Dense5, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x4096x4096, Dense4, rmsnorm_rope_bf16_512x4096, NormRopeW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(gemm_bf16_512x14336x4096, Dense7, rmsnorm_rope_bf16_512x4096, NormRopeW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(conv3x3_f32_128x28x28_128, Conv4, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(bgemm_f32_12x512x64x512, Bgemm0, softmax_causal_12x512x512, Softmax4W, _c256, bfuse::kChunked, 256, 1)
BFUSE_BFUSE_KERNEL(bgemm_f32_12x512x512x64, Bgemm1, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
