"""CPU-oracle evaluation of each synthetic pair (test side only)."""
import numpy as np

from oracle import oracle as orf


def expected(pair_number, I1, F1, I2, F2):
    """Returns (O1, O2) of the CPU reference for one pair."""
    if pair_number == 1:
        return (orf.gemm_f32(I1.reshape(512, 512), F1.reshape(512, 512)),
                orf.bias_relu(I2, F2))
    if pair_number == 2:
        return (orf.gemm_f32(I1.reshape(512, 768), F1.reshape(768, 2304)),
                orf.layernorm(I2.reshape(512, 768), F2[:768], F2[768:], 1e-12))
    if pair_number == 3:
        return (orf.conv2d(I1.reshape(1, 64, 56, 56), F1.reshape(64, 64, 3, 3), s=1, p=1),
                orf.maxpool2d(I2.reshape(1, 64, 112, 112), 3, 2, 1))
    if pair_number == 4:
        return (orf.softmax_causal(I1.reshape(12, 512, 512)),
                orf.gemm_f32(I2.reshape(512, 768), F2.reshape(768, 3072), epilogue=1))
    if pair_number == 5:
        # full-size bf16 GEMM takes minutes on the CPU: the oracle evaluates a strided sample
        # (every 8th row x every 8th column, 64 x 1792 outputs over the full K = 4096)
        from bfuse_project_amd.workloads import unpack_norm_rope_operand
        A, Wt = I1.reshape(512, 4096), F1.reshape(14336, 4096)
        rows, cols = np.arange(3, 512, 8), np.arange(5, 14336, 8)
        E1 = orf.gemm_bf16(np.ascontiguousarray(A[rows]), np.ascontiguousarray(Wt[cols]), b_is_nk=True)
        w, cosv, sinv = unpack_norm_rope_operand(F2, 512, 4096, 128)
        E2 = orf.rmsnorm_rope_bf16(I2.reshape(512, 4096), w, cosv, sinv, heads=32, eps=1e-5)
        return Sampled(E1, rows, cols, (512, 14336)), E2
    raise KeyError(pair_number)


class Sampled:
    """Expected values on a row/column sample of a matrix output."""

    def __init__(self, values, rows, cols, shape):
        self.values, self.rows, self.cols, self.shape = values, rows, cols, shape

    def pick(self, got):
        return np.ascontiguousarray(np.asarray(got).reshape(self.shape)[np.ix_(self.rows, self.cols)])


def rel_error(got, want):
    """Worst |got-want| / max(|want|, rms(want)): relative error against the reference value,
    measured against the output's RMS for elements smaller than it."""
    want = np.asarray(want, np.float32)
    rms = float(np.sqrt(np.mean(np.square(want.astype(np.float64)))))
    return orf.max_rel(got, want, rms)


def rel_stats(got, want, tol):
    """The acceptance rule next to the rule the configuration states ("relative").

    Accepted here: |got - want| <= tol * max(|want|, rms(want)).  Pure relative error has no meaning
    for outputs near zero (sums of ~K products of both signs cancel to values far below the size of
    the terms, and the rounding of the TERMS does not shrink with the sum), hence the RMS floor.
    Returned: the worst error under the accepted rule, the worst PURE relative error over the
    elements that are not tiny (|want| >= 1e-3 rms), and how many elements pass only thanks to the
    floor (pure relative error above tol)."""
    g = np.asarray(got, np.float64).ravel()
    w = np.asarray(want, np.float64).ravel()
    rms = float(np.sqrt(np.mean(w * w)))
    d = np.abs(g - w)
    floor = np.maximum(np.abs(w), rms)
    sizable = np.abs(w) >= 1e-3 * rms
    pure = np.where(np.abs(w) > 0, d / np.maximum(np.abs(w), 1e-300), np.where(d > 0, np.inf, 0.0))
    return {"n": int(g.size), "rms": rms, "worst_floor_rel": float((d / floor).max()),
            "worst_pure_rel_sizable": float(pure[sizable].max()) if sizable.any() else 0.0,
            "n_sizable": int(sizable.sum()),
            "n_pass_only_by_floor": int(((pure > tol) & (d <= tol * floor)).sum()),
            "n_fail": int((d > tol * floor).sum())}
