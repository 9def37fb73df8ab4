// The remaining operator ids of the reference's llm.yaml: the Llama-3-8B dense layers in fp32 (the
// reference's arithmetic; the bf16 instantiations are in kernels_models.hip and kernels_cfg5.hip),
// bgemm_4 .. bgemm_17, and the transposes that bring a dense weight from the reference's (out, in)
// layout into the [K, N] layout the fp32 GEMM sides take.  Each with a memory-bound partner,
// block-fused one chunk per round over the CUs.
#include "fuse.h"
#include "model_ops.h"
#include "ops_layout.h"

using namespace bfuse;
using namespace bfuse::model;

BFUSE_MODULE_PROLOGUE()

#define DENSE_F32(M, K, N, OP)                                                                                   \
    BFUSE_KERNEL(gemm_f32_##M##x##K##x##N, OP, ({{M, K, 1, 1}, 4}), ({{K, N, 1, 1}, 4}), ({{M, N, 1, 1}, 4}))      \
    BFUSE_BFUSE_KERNEL(gemm_f32_##M##x##K##x##N, OP, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
DENSE_F32(512, 4096, 4096, Dense4F32)
DENSE_F32(512, 4096, 14336, Dense6F32)
DENSE_F32(512, 14336, 4096, Dense7F32)

#define BGEMM_F32(B, M, K, N, OP)                                                                                \
    BFUSE_KERNEL(bgemm_f32_##B##x##M##x##K##x##N, OP, ({{B, M, K, 1}, 4}), ({{B, N, K, 1}, 4}), ({{B, M, N, 1}, 4})) \
    BFUSE_BFUSE_KERNEL(bgemm_f32_##B##x##M##x##K##x##N, OP, layernorm_512x768, LayerNormW1, _c256, bfuse::kChunked, 256, 1)
BGEMM_F32(16, 256, 64, 256, Bgemm4)
BGEMM_F32(16, 256, 256, 64, Bgemm5)
BGEMM_F32(16, 256, 80, 256, Bgemm6)
BGEMM_F32(16, 256, 256, 80, Bgemm7)
BGEMM_F32(16, 208, 64, 208, Bgemm8)
BGEMM_F32(16, 208, 208, 64, Bgemm9)
BGEMM_F32(16, 208, 80, 208, Bgemm10)
BGEMM_F32(16, 208, 208, 80, Bgemm11)
BGEMM_F32(1, 512, 64, 256, Bgemm12)
BGEMM_F32(1, 512, 256, 64, Bgemm13)
BGEMM_F32(1, 768, 64, 384, Bgemm14)
BGEMM_F32(1, 768, 384, 64, Bgemm15)
BGEMM_F32(1, 1024, 64, 512, Bgemm16)
BGEMM_F32(1, 1024, 512, 64, Bgemm17)

// dense weight (out, in) = [N, K]  ->  [K, N], once per weight: transpose32_<N>x<K>
#define WEIGHT_T(N, K)                                                                                           \
    using WeightT_##N##x##K = Transpose32<N, K>;                                                                 \
    BFUSE_KERNEL(transpose32_##N##x##K, WeightT_##N##x##K, ({{N, K, 1, 1}, 4}), ({{1, 1, 1, 1}, 4}), ({{K, N, 1, 1}, 4}))
WEIGHT_T(512, 512)
WEIGHT_T(768, 768)
WEIGHT_T(3072, 768)
WEIGHT_T(768, 3072)
WEIGHT_T(2304, 768)
WEIGHT_T(4096, 4096)
WEIGHT_T(1024, 4096)
WEIGHT_T(14336, 4096)
WEIGHT_T(4096, 14336)
