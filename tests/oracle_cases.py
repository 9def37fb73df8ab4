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
    raise KeyError(pair_number)


def rel_error(got, want):
    """Worst |got-want| / max(|want|, rms(want)): relative error against the reference value,
    measured against the output's RMS for elements smaller than it."""
    want = np.asarray(want, np.float32)
    rms = float(np.sqrt(np.mean(np.square(want.astype(np.float64)))))
    return orf.max_rel(got, want, rms)
