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


PAIRS: Dict[int, Pair] = {
    1: Pair(1, "GEMM fp32 512x512x512 || ReLU(x+b) over 1Mi fp32, hfuse 128/128",
            "gemm_f32_512x512x512", "bias_relu_1048576", "hfuse",
            [("hfuse", ""), ("bfuse", ""), ("bfuse", "_c8")], [], _pair1_inputs,
            bytes1=3 * 512 * 512 * 4, bytes2=3 * 1048576 * 4, flops=2 * 512 ** 3,
            bound="hbm", peak=8000.0, dtype="f32", tol=1e-5),
    2: Pair(2, "GEMM fp32 [512x768].[768x2304] || LayerNorm [512x768], bfuse",
            "gemm_f32_512x768x2304", "layernorm_512x768", "bfuse",
            [("bfuse", ""), ("bfuse", "_z2"), ("bfuse", "_c8"), ("bfuse", "_r")],
            [("gemm_f32_512x768x2304", "layernorm_512x768_w2", "bfuse", "_r"),
             ("gemm_f32_512x768x2304", "layernorm_512x768_w1", "bfuse", "_r"),
             ("gemm_f32_512x768x2304", "layernorm_512x768_w2", "hfuse", ""),
             ("gemm_f32_512x768x2304_p3", "layernorm_512x768_w2", "hfuse", ""),
             ("gemm_f32_512x768x2304_p3", "layernorm_512x768_w2", "bfuse", "_r")], _pair2_inputs,
            bytes1=(512 * 768 + 768 * 2304 + 512 * 2304) * 4, bytes2=(2 * 512 * 768 + 2 * 768) * 4,
            flops=2 * 512 * 768 * 2304, bound="mfma", peak=157.3, dtype="f32", tol=1e-5),
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
    2: ("gemm_f32_512x768x2304", "layernorm_512x768_w1", "bfuse", "_r"),
}
