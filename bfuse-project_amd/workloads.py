"""The five synthetic fused pairs: kernel names, seeded inputs, algorithmic work.

Inputs are generated on the host by the library's counter-based generator (element i of a
tensor depends only on (seed, i)); seed = 0xB5F05E + pair number, plus a per-tensor offset.
"""
from dataclasses import dataclass
from typing import Callable, Dict, List, Tuple

import numpy as np

from .operation import fill_normal, fill_uniform, f32_to_bf16

SEED0 = 0xB5F05E


@dataclass
class Pair:
    number: int
    title: str
    k1: str
    k2: str
    fusion: str                      # headline fused variant: "hfuse" | "bfuse"
    variants: List[Tuple[str, str]]  # every built (kind, suffix) of (k1, k2)
    alts: List[Tuple[str, str, str, str]]   # other built fusions of the same pair: (k1, k2, kind, suffix)
    inputs: Callable[[], Tuple[np.ndarray, np.ndarray, np.ndarray, np.ndarray]]   # I1, F1, I2, F2
    bytes1: int                      # algorithmic bytes of side 1 (operands read once + result written once)
    bytes2: int
    flops: int                       # contraction flops (2*M*N*K) of the GEMM / conv side
    bound: str                       # "hbm" | "mfma"
    peak: float                      # roofline ceiling for `bound` (GB/s or TFLOP/s)
    dtype: str
    tol: float                       # relative tolerance against the CPU reference


def _seed(pair, tensor):
    return (SEED0 + pair) * 16 + tensor


def _pair1_inputs():
    a = fill_uniform(_seed(1, 0), 512 * 512, -1.0, 1.0)
    b = fill_uniform(_seed(1, 1), 512 * 512, -1.0, 1.0)
    x = fill_normal(_seed(1, 2), 1048576, 0.0, 1.0)
    bias = fill_normal(_seed(1, 3), 1048576, 0.0, 0.1)
    return a, b, x, bias


def _pair2_inputs():
    a = fill_normal(_seed(2, 0), 512 * 768, 0.0, 1.0)
    w = fill_normal(_seed(2, 1), 768 * 2304, 0.0, 0.02)
    x = fill_normal(_seed(2, 2), 512 * 768, 0.0, 1.0)
    gb = np.concatenate([np.ones(768, np.float32), np.zeros(768, np.float32)])
    return a, w, x, gb


def _pair3_inputs():
    x = np.maximum(fill_normal(_seed(3, 0), 64 * 56 * 56, 0.0, 1.0), np.float32(0.0))
    w = fill_normal(_seed(3, 1), 64 * 64 * 9, 0.0, 0.05)
    p = fill_normal(_seed(3, 2), 64 * 112 * 112, 0.0, 1.0)
    unused = np.zeros(1, np.float32)
    return x, w, p, unused


def _pair4_inputs():
    scores = fill_normal(_seed(4, 0), 12 * 512 * 512, 0.0, 1.0) / np.float32(8.0)
    unused = np.zeros(1, np.float32)
    a = fill_normal(_seed(4, 2), 512 * 768, 0.0, 1.0)
    w = fill_normal(_seed(4, 3), 768 * 3072, 0.0, 0.02)
    return scores, unused, a, w


def rope_tables(S: int, hd: int, theta: float):
    """cos/sin tables [S, hd] of rotate-half RoPE: angle(p, j) = p * theta^(-2*(j mod hd/2)/hd),
    evaluated in double, stored fp32 (the Llama dump holds them as (1,1,S,hd) constants)."""
    j = np.arange(hd) % (hd // 2)
    inv = np.power(float(theta), -2.0 * j / hd)
    ang = np.arange(S, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


def pack_norm_rope_operand(w_bf16: np.ndarray, cosv: np.ndarray, sinv: np.ndarray) -> np.ndarray:
    """Second operand of the RMSNorm+RoPE kernel: weight (bf16), cos table, sin table (fp32), as bytes."""
    return np.concatenate([w_bf16.view(np.uint8).ravel(), cosv.view(np.uint8).ravel(), sinv.view(np.uint8).ravel()])


def unpack_norm_rope_operand(F: np.ndarray, S: int, d: int, hd: int):
    F = np.ascontiguousarray(F, np.uint8)
    w = F[: 2 * d].view(np.uint16)
    cosv = F[2 * d: 2 * d + 4 * S * hd].view(np.float32).reshape(S, hd)
    sinv = F[2 * d + 4 * S * hd:].view(np.float32).reshape(S, hd)
    return w, cosv, sinv


def _pair5_inputs():
    a = f32_to_bf16(fill_normal(_seed(5, 0), 512 * 4096, 0.0, 1.0))
    w = f32_to_bf16(fill_normal(_seed(5, 1), 14336 * 4096, 0.0, 0.02))       # [N, K] = (out, in)
    x = f32_to_bf16(fill_normal(_seed(5, 2), 512 * 4096, 0.0, 1.0))
    cosv, sinv = rope_tables(512, 128, 500000.0)
    f2 = pack_norm_rope_operand(f32_to_bf16(np.ones(4096, np.float32)), cosv, sinv)
    return a, w, x, f2


PAIRS: Dict[int, Pair] = {
    1: Pair(1, "GEMM fp32 512x512x512 || ReLU(x+b) over 1Mi fp32, hfuse 128/128",
            "gemm_f32_512x512x512", "bias_relu_1048576", "hfuse",
            [("hfuse", ""), ("bfuse", ""), ("bfuse", "_c8")],
            [("gemm_f32_512x512x512_k4", "bias_relu_1048576", "hfuse", "")], _pair1_inputs,
            bytes1=3 * 512 * 512 * 4, bytes2=3 * 1048576 * 4, flops=2 * 512 ** 3,
            bound="hbm", peak=8000.0, dtype="f32", tol=1e-5),
    2: Pair(2, "GEMM fp32 [512x768].[768x2304] || LayerNorm [512x768], bfuse",
            "gemm_f32_512x768x2304", "layernorm_512x768", "bfuse",
            [("bfuse", "_r"), ("bfuse", ""), ("bfuse", "_c8")],
            [("gemm_f32_512x768x2304_v", "layernorm_512x768", "bfuse", "_r"),
             ("gemm_f32_512x768x2304", "layernorm_512x768_w4", "bfuse", "_r")], _pair2_inputs,
            bytes1=(512 * 768 + 768 * 2304 + 512 * 2304) * 4, bytes2=(2 * 512 * 768 + 2 * 768) * 4,
            flops=2 * 512 * 768 * 2304, bound="mfma", peak=157.3, dtype="f32", tol=1e-5),
    3: Pair(3, "conv 3x3 s1 p1 [1,64,56,56]->64 fp32 || max-pool 3x3 s2 p1 [1,64,112,112], zig-zag bfuse",
            "conv3x3_f32_64x56x56_64", "maxpool3x3s2_f32_64x112x112", "bfuse",
            [("bfuse", "_c256"), ("bfuse", ""), ("bfuse", "_c8"), ("hfuse", "")],
            [], _pair3_inputs,
            bytes1=(64 * 56 * 56 * 2 + 64 * 64 * 9) * 4, bytes2=(64 * 112 * 112 + 64 * 56 * 56) * 4,
            flops=2 * 64 * 64 * 9 * 56 * 56, bound="mfma", peak=157.3, dtype="f32", tol=1e-5),
    4: Pair(4, "causal softmax 12x[512x512] fp32 || GEMM fp32 [512x768].[768x3072] + tanh-GELU, bfuse",
            "softmax_causal_12x512x512", "gemm_gelu_f32_512x768x3072", "bfuse",
            [("bfuse", "_c256"), ("bfuse", "_c512"), ("bfuse", "")],
            [("softmax_causal_12x512x512", "gemm_gelu_f32_512x768x3072_s3", "bfuse", "_c256"),
             ("softmax_causal_12x512x512_r3", "gemm_gelu_f32_512x768x3072", "hfuse", "")], _pair4_inputs,
            bytes1=2 * 12 * 512 * 512 * 4, bytes2=(512 * 768 + 768 * 3072 + 512 * 3072) * 4,
            flops=2 * 512 * 768 * 3072, bound="mfma", peak=157.3, dtype="f32", tol=1e-5),
    5: Pair(5, "GEMM bf16 [512x4096].[14336x4096]^T (fp32 acc) || RMSNorm+RoPE [512x4096] bf16, norm waves inside the GEMM workgroups",
            "gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096_w2", "hfuse",
            [("hfuse", "")],
            [("gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096", "bfuse", "_c256"),
             ("gemm_bf16_512x4096x14336_w8", "rmsnorm_rope_bf16_512x4096", "bfuse", "_c256"),
             ("gemm_bf16_512x4096x14336_w8", "rmsnorm_rope_bf16_512x4096", "bfuse", ""),
             ("gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096_w4", "bfuse", "_c256")], _pair5_inputs,
            bytes1=(512 * 4096 + 4096 * 14336 + 512 * 14336) * 2, bytes2=2 * 512 * 4096 * 2 + 4096 * 2,
            flops=2 * 512 * 4096 * 14336, bound="mfma", peak=2500.0, dtype="bf16", tol=1e-2),
}


def _qkv_ln_softmax_inputs():
    I1, F1, I2, F2 = _pair2_inputs()
    I3, F3, _, _ = _pair4_inputs()
    return [(I1, F1), (I2, F2), (I3, F3)]


# Fusions of more than two kernels (the reference's fuser takes a list of any length,
# horizontal-fuser/src/Algorithms.cc:23-35): name -> (standalone kernels, kind, suffixes built, inputs).
# One full-size group: the fp32 QKV projection, the LayerNorm and the causal softmax of pairs 2 and 4.
GROUPS = {
    "qkv_ln_softmax": (("gemm_f32_512x768x2304_s2", "layernorm_512x768", "softmax_causal_12x512x512"), "bfuse",
                       ("_c256", "_r"), _qkv_ln_softmax_inputs),
}


def fusions(pair: Pair):
    """Every built fusion of a pair, grouped by the two standalone kernels it fuses:
    {(k1, k2): [(kind, suffix), ...]}."""
    out = {(pair.k1, pair.k2): list(pair.variants)}
    for k1, k2, kind, suffix in pair.alts:
        out.setdefault((k1, k2), []).append((kind, suffix))
    return out


# headline fused variant of each pair: (k1, k2, kind, suffix)
HEADLINE = {
    1: ("gemm_f32_512x512x512", "bias_relu_1048576", "hfuse", ""),
    2: ("gemm_f32_512x768x2304", "layernorm_512x768", "bfuse", "_r"),
    3: ("conv3x3_f32_64x56x56_64", "maxpool3x3s2_f32_64x112x112", "bfuse", "_c256"),
    4: ("softmax_causal_12x512x512", "gemm_gelu_f32_512x768x3072", "bfuse", "_c256"),
    5: ("gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096_w2", "hfuse", ""),
}

# fused forms that the configurations name but that are not the fastest on this chip, timed beside the
# headline kernel: (label, k1, k2, kind, suffix)
BESIDE = {
    3: [("zigzag_1to1", "conv3x3_f32_64x56x56_64", "maxpool3x3s2_f32_64x112x112", "bfuse", "")],
    5: [("block_fused_chunk256", "gemm_bf16_512x4096x14336", "rmsnorm_rope_bf16_512x4096", "bfuse", "_c256")],
}

# fusion kinds the chooser picks from for each pair.  The configurations call pair 1 "horizontally
# fused" and pairs 2-5 "block-fused"; pair 5 is opened to both because block fusion cannot pay there
# (every workgroup of a block-fused kernel is charged the GEMM's 135 KB of LDS, so no norm workgroup
# ever shares a CU with a GEMM workgroup), and the block-fused kernel is timed beside it.
CONFIG_KINDS = {1: ("hfuse",), 2: ("bfuse",), 3: ("bfuse",), 4: ("bfuse",), 5: ("hfuse", "bfuse")}

# the pair whose block-fused kernel takes its dispatch plan at run time (`..._fused_bfuse_rt`), for the tuner
RT_SIDES = {
    1: ("gemm_f32_512x512x512", "bias_relu_1048576"),
    2: ("gemm_f32_512x768x2304", "layernorm_512x768"),
    3: ("conv3x3_f32_64x56x56_64", "maxpool3x3s2_f32_64x112x112"),
    4: ("softmax_causal_12x512x512", "gemm_gelu_f32_512x768x3072"),
    5: ("gemm_bf16_512x4096x14336_w8", "rmsnorm_rope_bf16_512x4096"),
}


# Bytes per launch that leave the eight L2s towards memory, for each headline fused kernel: measured
# with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE and scaled by what the same counters read for a 64 MiB
# copy kernel.  The figures live in the profile summaries shipped with the repository (derivation and
# commands are there); `measured_traffic` reads the fused kernel's row out of its summary, so the
# benchmark line cannot quote a figure the summary does not hold.  An operand that workgroups on all
# eight XCDs share is counted once per XCD.
TRAFFIC_SOURCE = {
    "gemm_f32_512x512x512_bias_relu_1048576_fused_hfuse": "profiles/pair1_gemm_f32_bias_relu_hfuse.md",
    "gemm_f32_512x768x2304_layernorm_512x768_fused_bfuse_r": "profiles/pair2_gemm_f32_layernorm_bfuse.md",
    "conv3x3_f32_64x56x56_64_maxpool3x3s2_f32_64x112x112_fused_bfuse_c256": "profiles/pair3_conv3x3_maxpool_bfuse.md",
    "softmax_causal_12x512x512_gemm_gelu_f32_512x768x3072_fused_bfuse_c256": "profiles/pair4_softmax_gemm_gelu_bfuse.md",
    "gemm_bf16_512x4096x14336_rmsnorm_rope_bf16_512x4096_w2_fused_hfuse": "profiles/pair5_gemm_bf16_rmsnorm_rope_hfuse.md",
}


def measured_traffic(kernel: str, root: str = None):
    """Bytes per launch of `kernel` from the traffic table of its profile summary (the row
    "| `kernel` | FETCH raw | WRITE raw | read MB | write MB | total MB |"), or None if the kernel has no
    summary.  Raises if the summary exists but holds no row for the kernel: the summary then describes another
    build."""
    import os
    src = TRAFFIC_SOURCE.get(kernel)
    if src is None:
        return None
    root = root or os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    with open(os.path.join(root, src)) as f:
        for line in f:
            cells = [c.strip() for c in line.split("|")]
            if len(cells) >= 8 and cells[1] == f"`{kernel}`":
                return int(round(float(cells[6]) * 1e6, -4))
    raise LookupError(f"{src} has no traffic row for {kernel}")


def check_traffic_sources(root: str = None) -> dict:
    """Every headline fused kernel is registered, has a profile summary, and the summary has its row.
    Part of the build check (__graft_entry__.build) and of the host tests."""
    from .operation import kernel_info
    out = {}
    for n, (k1, k2, kind, suffix) in HEADLINE.items():
        name = f"{k1}_{k2}_fused_{kind}{suffix}"
        kernel_info(name)                         # raises for a kernel the library does not hold
        if name not in TRAFFIC_SOURCE:
            raise LookupError(f"pair {n}: no profile summary is named for {name}")
        out[name] = measured_traffic(name, root)
    return out


def standalone_alternatives(name: str) -> List[str]:
    """Every standalone kernel of the registry that computes what `name` computes: the same operator at the
    same shapes (a variant suffix such as _s3, _k4, _w2 names another tiling or schedule of it)."""
    import re
    from .operation import kernel_info, list_kernels
    me = kernel_info(name)
    base = re.sub(r"_[a-z]+\d*$", "", name)
    out = []
    for k in list_kernels():
        if k.kind != 0 or (k.name != base and not re.fullmatch(re.escape(base) + r"_[a-z]+\d*", k.name)):
            continue
        if tuple(map(tuple, k.shapes)) == tuple(map(tuple, me.shapes)) and tuple(k.elem_bytes) == tuple(me.elem_bytes):
            out.append(k.name)
    return out


# Standalone kernels that are not a like-for-like baseline for a pair, with the reason (reported, still timed)
BASELINE_NOTES = {
    "gemm_f32_512x512x512_k4": "four waves split K: outside configuration 1's 128/128 thread split (its GEMM side is two waves)",
}

# what bounds a pair from below whatever the fusion does, stated in the benchmark line
FLOORS = {
    1: {"us": 3.9, "why": "the configuration's 128/128 thread split gives the GEMM side two waves = two of a CU's four SIMDs; "
                          "256 MFMAs of 32 clocks on each = 8192 clocks = 3.9 us at 2.1 GHz, before launch and memory latency; "
                          "the element-wise side finishes inside it (fused = GEMM alone + 0.1 us)"},
}
