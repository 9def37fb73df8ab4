"""ctypes binding of include/bfuse_rt.h."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libbfuse_rt.so")

MAXK, MAXSEG = 4, 8


class LibraryMissing(RuntimeError):
    pass


class BfuseError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"libbfuse_rt error {code}: {text}")
        self.code = code


class LaunchDimsC(C.Structure):
    _fields_ = [("grid", C.c_int * 3), ("block", C.c_int * 3)]


class SlotC(C.Structure):
    _fields_ = [("kern", C.c_int), ("off", C.c_int), ("width", C.c_int), ("base", C.c_int)]


class SegmentC(C.Structure):
    _fields_ = [("lo", C.c_int), ("hi", C.c_int), ("period", C.c_int), ("n_slot", C.c_int), ("slot", SlotC * MAXK)]


class BlockPlanC(C.Structure):
    _fields_ = [("n_kernels", C.c_int), ("n_seg", C.c_int), ("seg", SegmentC * MAXSEG),
                ("fused_grid", C.c_int), ("fused_block", C.c_int), ("threads", C.c_int * MAXK)]


class ThreadPlanC(C.Structure):
    _fields_ = [("n_kernels", C.c_int), ("thr_lo", C.c_int * MAXK), ("thr_hi", C.c_int * MAXK),
                ("blocks", C.c_int * MAXK), ("fused_grid", C.c_int), ("fused_block", C.c_int)]


class KernelInfoC(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("func", C.c_void_p), ("kind", C.c_int),
                ("grid", C.c_uint * 3), ("block", C.c_uint * 3), ("has_barriers", C.c_int),
                ("regs", C.c_int), ("lds_bytes", C.c_int), ("shape", (C.c_int * 4) * 3),
                ("elem_bytes", C.c_int * 3), ("side", (C.c_char * 64) * 2),
                ("pattern", C.c_int), ("p0", C.c_int), ("p1", C.c_int),
                ("n_sides", C.c_int), ("side_more", (C.c_char * 64) * (MAXK - 2)), ("matrix_cores", C.c_int)]


class LaunchDescC(C.Structure):
    _fields_ = [("func", C.c_void_p), ("grid", C.c_uint * 3), ("block", C.c_uint * 3),
                ("n_sides", C.c_int), ("sides", C.c_int * MAXK)]


# every symbol include/bfuse_rt.h declares
EXPORTS = [
    "bfuse_last_error", "bfuse_init", "bfuse_shutdown", "bfuse_device_info", "bfuse_device_memory",
    "bfuse_plan_threads", "bfuse_plan_blocks", "bfuse_map_block", "bfuse_map_thread", "bfuse_map_blocks_device", "bfuse_map_blocks_device_noalloc", "bfuse_probe_placement", "bfuse_set_plan",
    "bfuse_set_sync_spin_limit",
    "bfuse_kernel_count", "bfuse_kernel_at", "bfuse_kernel_find", "bfuse_load_kernels", "bfuse_kernel_op_type", "bfuse_kernel_op_lds",
    "bfuse_set_elem_bytes", "initialize_kernel1", "initialize_kernel2", "finalize_kernel1", "finalize_kernel2",
    "run_kernel1", "run_kernel2", "run_parallel", "run_fuse",
    "bfuse_upload", "bfuse_zero_output", "bfuse_download", "bfuse_synchronize", "bfuse_launch",
    "bfuse_upload_part", "bfuse_download_part", "bfuse_checksum_output", "bfuse_fill_uniform_device",
    "bfuse_time", "bfuse_time_batched", "bfuse_time_graph", "bfuse_module_load", "bfuse_module_unload", "bfuse_module_launch",
    "bfuse_initialize_side", "bfuse_finalize_side", "bfuse_launch_list", "bfuse_time_list",
    "bfuse_fill_uniform", "bfuse_fill_normal", "bfuse_f32_to_bf16", "bfuse_bf16_to_f32", "bfuse_check_matrix",
]

_LIB = None


def lib():
    """Loads libbfuse_rt.so; raises LibraryMissing if it has not been built (no fallback)."""
    global _LIB
    if _LIB is None:
        if not os.path.exists(LIB_PATH):
            raise LibraryMissing(
                f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "or `make -C bfuse-project_amd/csrc` (hipcc, gfx950)")
        l = C.CDLL(LIB_PATH)
        l.bfuse_last_error.restype = C.c_char_p
        l.bfuse_check_matrix.restype = C.c_long
        l.bfuse_check_matrix.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float]
        l.bfuse_fill_uniform.restype = None
        l.bfuse_fill_uniform.argtypes = [C.c_ulonglong, C.c_size_t, C.c_float, C.c_float, C.c_void_p]
        l.bfuse_fill_normal.restype = None
        l.bfuse_fill_normal.argtypes = [C.c_ulonglong, C.c_size_t, C.c_float, C.c_float, C.c_void_p]
        l.bfuse_f32_to_bf16.restype = None
        l.bfuse_f32_to_bf16.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p]
        l.bfuse_bf16_to_f32.restype = None
        l.bfuse_bf16_to_f32.argtypes = [C.c_size_t, C.c_void_p, C.c_void_p]
        ip, up, vp = C.POINTER(C.c_int), C.POINTER(C.c_uint), C.c_void_p
        l.bfuse_device_info.argtypes = [C.c_char_p, C.c_size_t, ip, ip, ip]
        l.bfuse_plan_threads.argtypes = [C.c_int, C.POINTER(LaunchDimsC), C.c_int, C.POINTER(ThreadPlanC)]
        l.bfuse_plan_blocks.argtypes = [C.c_int, C.c_int, C.POINTER(LaunchDimsC), C.c_int, C.c_int, C.POINTER(BlockPlanC)]
        l.bfuse_map_block.argtypes = [C.POINTER(BlockPlanC), C.c_int, ip]
        l.bfuse_map_thread.argtypes = [C.POINTER(ThreadPlanC), C.c_int, C.c_int, ip]
        l.bfuse_map_blocks_device.argtypes = [C.POINTER(BlockPlanC), C.c_int, C.c_int, vp, vp]
        l.bfuse_map_blocks_device_noalloc.argtypes = [C.POINTER(BlockPlanC), C.c_int, C.c_int, vp, vp]
        l.bfuse_set_plan.argtypes = [vp, C.POINTER(BlockPlanC)]
        l.bfuse_set_sync_spin_limit.argtypes = [vp, C.c_uint]
        l.bfuse_probe_placement.argtypes = [C.c_int, C.c_int, C.c_int, vp, vp, vp, vp, vp]
        l.bfuse_kernel_at.argtypes = [C.c_int, C.POINTER(KernelInfoC)]
        l.bfuse_kernel_find.argtypes = [C.c_char_p, C.POINTER(KernelInfoC)]
        l.bfuse_load_kernels.argtypes = [C.c_char_p]
        l.bfuse_kernel_op_type.argtypes = [C.c_char_p]
        l.bfuse_kernel_op_type.restype = C.c_char_p
        l.bfuse_kernel_op_lds.argtypes = [C.c_char_p]
        for n in ("initialize_kernel1", "initialize_kernel2"):
            getattr(l, n).argtypes = [ip, ip, ip]
        for n in ("run_kernel1", "run_kernel2"):
            getattr(l, n).argtypes = [vp, vp, vp, ip, ip, ip, vp, up, up, C.c_size_t]
        l.run_parallel.argtypes = [vp] * 6 + [ip] * 6 + [vp, vp, up, up, up, up, C.c_size_t, C.c_size_t]
        l.run_fuse.argtypes = [vp] * 6 + [ip] * 6 + [vp, up, up, C.c_size_t, C.c_size_t]
        l.bfuse_upload.argtypes = [C.c_int, vp, vp]
        l.bfuse_download.argtypes = [C.c_int, vp]
        l.bfuse_upload_part.argtypes = [C.c_int, C.c_int, C.c_size_t, vp, C.c_size_t]
        l.bfuse_download_part.argtypes = [C.c_int, C.c_size_t, vp, C.c_size_t]
        l.bfuse_checksum_output.argtypes = [C.c_int, C.c_size_t, vp]
        l.bfuse_fill_uniform_device.argtypes = [C.c_int, C.c_int, C.c_ulonglong, C.c_float, C.c_float]
        l.bfuse_launch.argtypes = [C.c_int, vp, up, up, vp, up, up]
        fp = C.POINTER(C.c_float)
        l.bfuse_time.argtypes = [C.c_int, vp, up, up, vp, up, up, C.c_int, C.c_int, fp, fp, fp]
        l.bfuse_time_batched.argtypes = [C.c_int, vp, up, up, vp, up, up, C.c_int, C.c_int, fp]
        l.bfuse_time_graph.argtypes = [C.c_int, vp, up, up, vp, up, up, C.c_int, C.c_int, fp]
        l.bfuse_initialize_side.argtypes = [C.c_int, ip, ip, ip]
        l.bfuse_finalize_side.argtypes = [C.c_int]
        l.bfuse_launch_list.argtypes = [C.c_int, C.POINTER(LaunchDescC)]
        l.bfuse_time_list.argtypes = [C.c_int, C.POINTER(LaunchDescC), C.c_int, C.c_int, fp, fp]
        l.bfuse_module_load.argtypes = [C.c_char_p, ip]
        l.bfuse_module_launch.argtypes = [C.c_int, C.c_char_p, up, up, C.c_int, C.c_int, fp]
        _LIB = l
    return _LIB


def check(rc):
    if rc != 0:
        raise BfuseError(rc, lib().bfuse_last_error().decode())
    return rc
