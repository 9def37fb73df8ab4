// Thread-level fusion for the pairs of the model-operator matrix whose grids allow it: a dense layer of one
// tile per CU (256 workgroups) with a convolution of 196 workgroups -- one fused workgroup per CU hosts a GEMM
// tile on four waves and a convolution tile on four more, LDS is the sum of the two sides.  Both sides
// synchronise only when their partial tiles meet, each on its own LDS arrival counter.
#include "fuse.h"
#include "model_ops.h"

using namespace bfuse;
using namespace bfuse::model;

BFUSE_MODULE_PROLOGUE()

BFUSE_HFUSE_KERNEL(gemm_f32_512x768x768, Dense0, conv3x3_f32_64x56x56_64, Conv1)
BFUSE_HFUSE_KERNEL(gemm_f32_512x768x768, Dense0, conv3x3_f32_128x28x28_128, Conv4)
BFUSE_HFUSE_KERNEL(gemm_f32_512x3072x768, Dense2, conv3x3_f32_64x56x56_64, Conv1)
BFUSE_HFUSE_KERNEL(gemm_f32_512x3072x768, Dense2, conv3x3_f32_128x28x28_128, Conv4)
BFUSE_HFUSE_KERNEL(gemm_f32_512x768x2304, Dense3, conv3x3_f32_64x56x56_64, Conv1)
BFUSE_HFUSE_KERNEL(gemm_f32_512x768x2304, Dense3, conv3x3_f32_128x28x28_128, Conv4)
BFUSE_HFUSE_KERNEL(gemm_f32_512x4096x1024, Dense5, conv3x3_f32_64x56x56_64, Conv1)
BFUSE_HFUSE_KERNEL(gemm_f32_512x4096x1024, Dense5, conv3x3_f32_128x28x28_128, Conv4)
