"""bfuse-project_amd: MI355X-native fused-pair runtime (host-side Python mirror).

The package is a thin ctypes layer over libbfuse_rt.so (HIP, gfx950).  There is no CPU
fallback: loading fails loudly if the library has not been built, and every device entry
point fails if no GPU is present.
"""
from ._lib import lib, LibraryMissing, BfuseError  # noqa: F401
from .patterns import (  # noqa: F401
    LaunchDims, plan_threads, plan_blocks, PATTERNS,
)
from .config import KernelInfo, FusionInfo, load_kernels_yaml, load_fusions_yaml, dump_kernels_yaml, FusionContext  # noqa: F401
from .operation import Operation, GroupOperation, kernel_info, list_kernels  # noqa: F401
