"""ctypes loader for liboracle.so -- TEST INFRASTRUCTURE ONLY.

Imported by tests/, by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py,
always as the checker; the product package never imports it.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build():
    subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = C.CDLL(path)
        _LIB.ork_check_matrix.restype = C.c_long
        _LIB.orf_count_rel.restype = C.c_long
        _LIB.orf_max_rel.restype = C.c_double
    return _LIB


def _ip(a):
    return a.ctypes.data_as(C.POINTER(C.c_int))


def _fp(a):
    return a.ctypes.data_as(C.POINTER(C.c_float))


def _hp(a):
    return a.ctypes.data_as(C.POINTER(C.c_uint16))


def _i32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.int32))


def _f32(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.float32))


def _u16(x):
    return np.ascontiguousarray(np.asarray(x, dtype=np.uint16))


# ---- index maps -----------------------------------------------------------------------
def hfuse_dims(grids, blocks, pad=32):
    g, b = _i32(grids).reshape(-1, 3), _i32(blocks).reshape(-1, 3)
    n = g.shape[0]
    lo, hi = np.zeros(n, np.int32), np.zeros(n, np.int32)
    fg, fb = C.c_int(), C.c_int()
    rc = lib().ork_hfuse_dims(n, _ip(g), _ip(b), pad, _ip(lo), _ip(hi), C.byref(fg), C.byref(fb))
    assert rc == 0
    return lo.tolist(), hi.tolist(), fg.value, fb.value


def hfuse_map(grids, blocks, pad, bid, tid):
    g, b = _i32(grids).reshape(-1, 3), _i32(blocks).reshape(-1, 3)
    vb, vt = np.zeros(3, np.int32), np.zeros(3, np.int32)
    k = lib().ork_hfuse_map(g.shape[0], _ip(g), _ip(b), pad, bid, tid, _ip(vb), _ip(vt))
    return k, vb.tolist(), vt.tolist()


def bfuse_dims(grids, blocks):
    g, b = _i32(grids).reshape(-1, 3), _i32(blocks).reshape(-1, 3)
    fg, fb = C.c_int(), C.c_int()
    lib().ork_bfuse_dims(g.shape[0], _ip(g), _ip(b), C.byref(fg), C.byref(fb))
    return fg.value, fb.value


KIND = {"zigzag": 0, "prop": 1, "chunk": 2}


def map_table(kind, gsizes, p0, p1=1, lo=0, hi=None):
    g = _i32(gsizes)
    if hi is None:
        hi = int(g.sum())
    k = np.empty(hi - lo, np.int32)
    v = np.empty(hi - lo, np.int32)
    rc = lib().ork_map_table(KIND[kind], len(g), _ip(g), int(p0), int(p1), lo, hi, _ip(k), _ip(v))
    assert rc == 0
    return k, v


def virtual_ids(grid, block, new_block_idx, tid):
    vb, vt = np.zeros(3, np.int32), np.zeros(3, np.int32)
    lib().ork_virtual_ids(_ip(_i32(grid)), _ip(_i32(block)), new_block_idx, tid, _ip(vb), _ip(vt))
    return vb.tolist(), vt.tolist()


def check_matrix(o, o_ans, eps=1e-3):
    o, a = _f32(o).ravel(), _f32(o_ans).ravel()
    assert o.size == a.size
    return lib().ork_check_matrix(_fp(o), _fp(a), C.c_long(o.size), C.c_float(eps))


# ---- operator references ---------------------------------------------------------------
def num_threads():
    return lib().orf_num_threads()


def f32_to_bf16(x):
    x = _f32(x)
    y = np.empty(x.shape, np.uint16)
    lib().orf_f32_to_bf16(C.c_long(x.size), _fp(x), _hp(y))
    return y


def bf16_to_f32(x):
    x = _u16(x)
    y = np.empty(x.shape, np.float32)
    lib().orf_bf16_to_f32(C.c_long(x.size), _hp(x), _fp(y))
    return y


def gemm_f32(A, B, b_is_nk=False, epilogue=0):
    A, B = _f32(A), _f32(B)
    M, K = A.shape
    N = B.shape[0] if b_is_nk else B.shape[1]
    assert (B.shape[1] if b_is_nk else B.shape[0]) == K
    Cm = np.empty((M, N), np.float32)
    lib().orf_gemm_f32(M, N, K, _fp(A), _fp(B), _fp(Cm), int(b_is_nk), int(epilogue))
    return Cm


def gemm_bf16(A, B, b_is_nk=False):
    A, B = _u16(A), _u16(B)
    M, K = A.shape
    N = B.shape[0] if b_is_nk else B.shape[1]
    Cm = np.empty((M, N), np.uint16)
    lib().orf_gemm_bf16(M, N, K, _hp(A), _hp(B), _hp(Cm), int(b_is_nk))
    return Cm


def bias_relu(x, b):
    x, b = _f32(x), _f32(b)
    y = np.empty_like(x)
    lib().orf_bias_relu(C.c_long(x.size), _fp(x), _fp(b), _fp(y))
    return y


def layernorm(x, gamma, beta, eps):
    x, gamma, beta = _f32(x), _f32(gamma), _f32(beta)
    y = np.empty_like(x)
    lib().orf_layernorm(x.shape[0], x.shape[1], _fp(x), _fp(gamma), _fp(beta), C.c_float(eps), _fp(y))
    return y


def maxpool2d(x, k=3, s=2, p=1):
    x = _f32(x)
    N, Cc, H, W = x.shape
    OH, OW = (H + 2 * p - k) // s + 1, (W + 2 * p - k) // s + 1
    y = np.empty((N, Cc, OH, OW), np.float32)
    lib().orf_maxpool2d(N, Cc, H, W, k, s, p, _fp(x), _fp(y))
    return y


def conv2d(x, w, s=1, p=1):
    x, w = _f32(x), _f32(w)
    N, CI, H, W = x.shape
    CO, CI2, KH, KW = w.shape
    assert CI == CI2
    OH, OW = (H + 2 * p - KH) // s + 1, (W + 2 * p - KW) // s + 1
    y = np.empty((N, CO, OH, OW), np.float32)
    lib().orf_conv2d(N, CI, H, W, CO, KH, KW, s, p, _fp(x), _fp(w), _fp(y))
    return y


def softmax_causal(x):
    x = _f32(x)
    heads, S, S2 = x.shape
    assert S == S2
    y = np.empty_like(x)
    lib().orf_softmax_causal(heads, S, _fp(x), _fp(y))
    return y


def rope_tables(S, hd, theta):
    c, s = np.empty((S, hd), np.float32), np.empty((S, hd), np.float32)
    lib().orf_rope_tables(S, hd, C.c_double(theta), _fp(c), _fp(s))
    return c, s


def rmsnorm_rope_bf16(x, w, cosv, sinv, heads, eps):
    x, w = _u16(x), _u16(w)
    S, d = x.shape
    hd = d // heads
    y = np.empty_like(x)
    lib().orf_rmsnorm_rope_bf16(S, heads, hd, _hp(x), _hp(w), _fp(_f32(cosv)), _fp(_f32(sinv)),
                                C.c_float(eps), _hp(y))
    return y


def count_rel(o, a, tol, floor_mag):
    o, a = _f32(o).ravel(), _f32(a).ravel()
    assert o.size == a.size
    return lib().orf_count_rel(C.c_long(o.size), _fp(o), _fp(a), C.c_double(tol), C.c_double(floor_mag))


def max_rel(o, a, floor_mag):
    o, a = _f32(o).ravel(), _f32(a).ravel()
    assert o.size == a.size
    return lib().orf_max_rel(C.c_long(o.size), _fp(o), _fp(a), C.c_double(floor_mag))
