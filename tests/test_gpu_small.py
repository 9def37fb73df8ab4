"""Parity of every operator body and fusion form on small shapes the CPU oracle evaluates in
full (needs the MI355X; everything goes through the C ABI).

fp32 tolerance: |gpu - ref| <= 1e-5 * max(|ref|, rms(ref)); bf16: 1e-2 likewise.
Fused outputs must equal the unfused ones bit for bit.
"""
import sys

import numpy as np
import pytest

import bfuse_project_amd as bf
from bfuse_project_amd import workloads as wl
from bfuse_project_amd.operation import fill_normal, fill_uniform, f32_to_bf16, bf16_to_f32
from oracle import oracle as orf
from tests.oracle_cases import rel_error

pytestmark = pytest.mark.gpu


def _say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def _norm_rope_operand(S, d, hd, seed):
    cosv, sinv = wl.rope_tables(S, hd, 500000.0)
    w = f32_to_bf16(fill_normal(seed, d, 1.0, 0.1))
    return wl.pack_norm_rope_operand(w, cosv, sinv)


# name -> (inputs(seed) -> (I, F), oracle(I, F) -> O, tolerance, is_bf16)
def _cases():
    z = np.zeros(1, np.float32)
    return {
        "gemm_f32_64x32x48": (lambda s: (fill_uniform(s, 64 * 32, -1, 1), fill_uniform(s + 1, 32 * 48, -1, 1)),
                              lambda I, F: orf.gemm_f32(I.reshape(64, 32), F.reshape(32, 48)), 1e-5, False),
        "gemm_f32_256x32x64_t128": (lambda s: (fill_uniform(s, 256 * 32, -1, 1), fill_uniform(s + 1, 32 * 64, -1, 1)),
                                    lambda I, F: orf.gemm_f32(I.reshape(256, 32), F.reshape(32, 64)), 1e-5, False),
        "gemm_f32_80x32x112": (lambda s: (fill_uniform(s, 80 * 32, -1, 1), fill_uniform(s + 1, 32 * 112, -1, 1)),
                               lambda I, F: orf.gemm_f32(I.reshape(80, 32), F.reshape(32, 112)), 1e-5, False),
        "bgemm_f32_3x48x64x80": (lambda s: (fill_uniform(s, 3 * 48 * 64, -1, 1), fill_uniform(s + 1, 3 * 80 * 64, -1, 1)),
                                 lambda I, F: np.stack([orf.gemm_f32(I.reshape(3, 48, 64)[b], F.reshape(3, 80, 64)[b], b_is_nk=True) for b in range(3)]), 1e-5, False),
        "gemm_gelu_f32_96x128x192": (lambda s: (fill_normal(s, 96 * 128, 0, 1), fill_normal(s + 1, 128 * 192, 0, 0.1)),
                                     lambda I, F: orf.gemm_f32(I.reshape(96, 128), F.reshape(128, 192), epilogue=1), 1e-5, False),
        "gemm_f32_32x256x144": (lambda s: (fill_normal(s, 32 * 256, 0, 1), fill_normal(s + 1, 256 * 144, 0, 0.05)),
                                lambda I, F: orf.gemm_f32(I.reshape(32, 256), F.reshape(256, 144)), 1e-5, False),
        "gemm_f32_128x160x192_d": (lambda s: (fill_normal(s, 128 * 160, 0, 1), fill_normal(s + 1, 160 * 192, 0, 0.1)),
                                   lambda I, F: orf.gemm_f32(I.reshape(128, 160), F.reshape(160, 192)), 1e-5, False),
        "gemm_gelu_f32_64x192x288_d": (lambda s: (fill_normal(s, 64 * 192, 0, 1), fill_normal(s + 1, 192 * 288, 0, 0.1)),
                                       lambda I, F: orf.gemm_f32(I.reshape(64, 192), F.reshape(192, 288), epilogue=1), 1e-5, False),
        "bias_relu_4096": (lambda s: (fill_normal(s, 4096, 0, 1), fill_normal(s + 1, 4096, 0, 0.1)),
                           lambda I, F: orf.bias_relu(I, F), 0.0, False),
        "layernorm_8x256": (lambda s: (fill_normal(s, 8 * 256, 0.5, 2), np.concatenate([fill_normal(s + 1, 256, 1, 0.1), fill_normal(s + 2, 256, 0, 0.1)])),
                            lambda I, F: orf.layernorm(I.reshape(8, 256), F[:256], F[256:], 1e-12), 1e-5, False),
        "softmax_causal_2x256x256": (lambda s: (fill_normal(s, 2 * 256 * 256, 0, 1) / np.float32(8), z),
                                     lambda I, F: orf.softmax_causal(I.reshape(2, 256, 256)), 1e-5, False),
        "conv3x3_f32_16x8x8_16": (lambda s: (np.maximum(fill_normal(s, 16 * 64, 0, 1), 0), fill_normal(s + 1, 16 * 16 * 9, 0, 0.05)),
                                  lambda I, F: orf.conv2d(I.reshape(1, 16, 8, 8), F.reshape(16, 16, 3, 3)), 1e-5, False),
        "conv3x3_f32_32x12x12_32": (lambda s: (np.maximum(fill_normal(s, 32 * 144, 0, 1), 0), fill_normal(s + 1, 32 * 32 * 9, 0, 0.05)),
                                    lambda I, F: orf.conv2d(I.reshape(1, 32, 12, 12), F.reshape(32, 32, 3, 3)), 1e-5, False),
        "conv3x3_f32_64x8x16_16": (lambda s: (fill_normal(s, 64 * 128, 0, 1), fill_normal(s + 1, 16 * 64 * 9, 0, 0.05)),
                                   lambda I, F: orf.conv2d(I.reshape(1, 64, 8, 16), F.reshape(16, 64, 3, 3)), 1e-5, False),
        "conv1x1s1p0_f32_3x32x5x5_32": (lambda s: (fill_normal(s, 3 * 32 * 25, 0, 1), fill_normal(s + 1, 32 * 32, 0, 0.2)),
                                        lambda I, F: orf.conv2d(I.reshape(3, 32, 5, 5), F.reshape(32, 32, 1, 1), s=1, p=0), 1e-5, False),
        "conv1x1s1p0_f32_5x96x9x9_48": (lambda s: (fill_normal(s, 5 * 96 * 81, 0, 1), fill_normal(s + 1, 48 * 96, 0, 0.1)),
                                        lambda I, F: orf.conv2d(I.reshape(5, 96, 9, 9), F.reshape(48, 96, 1, 1), s=1, p=0), 1e-5, False),
        "conv1x1s2p0_f32_2x16x9x7_16": (lambda s: (fill_normal(s, 2 * 16 * 63, 0, 1), fill_normal(s + 1, 16 * 16, 0, 0.25)),
                                        lambda I, F: orf.conv2d(I.reshape(2, 16, 9, 7), F.reshape(16, 16, 1, 1), s=2, p=0), 1e-5, False),
        "maxpool3x3s2_f32_4x16x16": (lambda s: (fill_normal(s, 4 * 256, -3, 1), z),        # all-negative: padding must not win
                                     lambda I, F: orf.maxpool2d(I.reshape(1, 4, 16, 16)), 0.0, False),
        "gemm_bf16_128x64x1792": (lambda s: (f32_to_bf16(fill_normal(s, 128 * 64, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1792 * 64, 0, 0.1))),
                                  lambda I, F: orf.gemm_bf16(I.reshape(128, 64), F.reshape(1792, 64), b_is_nk=True), 1e-2, True),
        "gemm_bf16_128x192x1792": (lambda s: (f32_to_bf16(fill_normal(s, 128 * 192, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1792 * 192, 0, 0.1))),
                                   lambda I, F: orf.gemm_bf16(I.reshape(128, 192), F.reshape(1792, 192), b_is_nk=True), 1e-2, True),
        "gemm_bf16_256x320x1792": (lambda s: (f32_to_bf16(fill_normal(s, 256 * 320, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1792 * 320, 0, 0.1))),
                                   lambda I, F: orf.gemm_bf16(I.reshape(256, 320), F.reshape(1792, 320), b_is_nk=True), 1e-2, True),
        "gemm_bf16_256x320x1792_w8": (lambda s: (f32_to_bf16(fill_normal(s, 256 * 320, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1792 * 320, 0, 0.1))),
                                      lambda I, F: orf.gemm_bf16(I.reshape(256, 320), F.reshape(1792, 320), b_is_nk=True), 1e-2, True),
        "gemm_bf16_256x384x1792_p": (lambda s: (f32_to_bf16(fill_normal(s, 256 * 384, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1792 * 384, 0, 0.1))),
                                     lambda I, F: orf.gemm_bf16(I.reshape(256, 384), F.reshape(1792, 384), b_is_nk=True), 1e-2, True),
        "gemm_bf16_256x448x1792_p2": (lambda s: (f32_to_bf16(fill_normal(s, 256 * 448, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1792 * 448, 0, 0.1))),
                                      lambda I, F: orf.gemm_bf16(I.reshape(256, 448), F.reshape(1792, 448), b_is_nk=True), 1e-2, True),
        "gemm_bf16_128x320x1024_t64": (lambda s: (f32_to_bf16(fill_normal(s, 128 * 320, 0, 1)), f32_to_bf16(fill_normal(s + 1, 1024 * 320, 0, 0.1))),
                                       lambda I, F: orf.gemm_bf16(I.reshape(128, 320), F.reshape(1024, 320), b_is_nk=True), 1e-2, True),
        "rmsnorm_rope_bf16_6x1024": (lambda s: (f32_to_bf16(fill_normal(s, 6 * 1024, 0, 1.5)), _norm_rope_operand(6, 1024, 128, s + 1)),
                                     lambda I, F: orf.rmsnorm_rope_bf16(I.reshape(6, 1024), *wl.unpack_norm_rope_operand(F, 6, 1024, 128), heads=8, eps=1e-5), 1e-2, True),
    }


FUSIONS = [
    ("gemm_gelu_f32_96x128x192", "bias_relu_4096", "hfuse", ""),
    ("gemm_gelu_f32_96x128x192", "conv3x3_f32_32x12x12_32", "hfuse", ""),
    ("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192", "bfuse", ""),
    ("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192", "bfuse", "_p1"),
    ("conv3x3_f32_32x12x12_32", "gemm_gelu_f32_96x128x192", "bfuse", "_c4"),
    ("layernorm_8x256", "softmax_causal_2x256x256", "bfuse", ""),
    ("gemm_bf16_256x320x1792", "rmsnorm_rope_bf16_6x1024", "bfuse", "_c8"),
    ("maxpool3x3s2_f32_4x16x16", "layernorm_8x256", "hfuse", ""),
    ("gemm_f32_128x160x192_d", "bias_relu_4096", "hfuse", ""),
    ("gemm_gelu_f32_64x192x288_d", "layernorm_8x256", "bfuse", "_c4"),
    ("gemm_bf16_256x320x1792_w8", "gemm_f32_128x160x192_d", "hfuse", ""),     # a barrier in the K loop, both sides synchronise: LDS arrival counters
    ("gemm_bf16_256x384x1792_p", "rmsnorm_rope_bf16_6x1024", "hfuse", ""),    # the norm waves join the GEMM's hardware loop barriers
    ("gemm_bf16_256x448x1792_p2", "rmsnorm_rope_bf16_6x1024", "hfuse", ""),   # the same with two producer waves (twelve waves in all)
    ("gemm_f32_128x160x192_d", "gemm_gelu_f32_64x192x288_d", "hfuse", ""),    # both sides synchronise: LDS arrival counters
    ("conv3x3_f32_32x12x12_32", "bias_relu_4096", "hfuse", ""),
    ("conv3x3_f32_64x8x16_16", "layernorm_8x256", "bfuse", "_c4"),
    ("conv1x1s1p0_f32_3x32x5x5_32", "layernorm_8x256", "bfuse", "_c4"),
    ("conv1x1s1p0_f32_5x96x9x9_48", "bias_relu_4096", "hfuse", ""),                # a barrier per filter chunk beside a side without any: LDS arrival counters
    ("conv1x1s1p0_f32_5x96x9x9_48", "conv3x3_f32_32x12x12_32", "hfuse", ""),       # both sides synchronise
    ("conv1x1s2p0_f32_2x16x9x7_16", "bias_relu_4096", "bfuse", ""),
    ("gemm_f32_256x32x64_t128", "bias_relu_4096", "bfuse", ""),                    # a side of 128 x 64 tiles: the fused kernels are kernels of one wave per SIMD
    ("gemm_f32_256x32x64_t128", "bias_relu_4096", "hfuse", ""),
    ("gemm_f32_80x32x112", "layernorm_8x256", "bfuse", ""),                        # GEMM tiles that overlap (80 = 32 + 32 + 16 rows)
    ("bgemm_f32_3x48x64x80", "bias_relu_4096", "hfuse", ""),
]


def _check(name, got, want, tol, is_bf16):
    if is_bf16:
        got, want = bf16_to_f32(got), bf16_to_f32(want)
    if tol == 0.0:
        assert np.array_equal(np.asarray(got).ravel(), np.asarray(want).ravel()), name
        return 0.0
    e = rel_error(np.asarray(got).ravel(), np.asarray(want).ravel())
    assert e <= tol, f"{name}: max rel err {e:.3e} > {tol:g}"
    return e


def test_every_small_operator_against_the_oracle():
    cases = _cases()
    names = sorted(cases)
    # kernels are run in (side1, side2) couples; the partner is just the next one in the list
    for i, name in enumerate(names):
        partner = names[(i + 1) % len(names)]
        gen, oracle, tol, is_bf16 = cases[name]
        I, F = gen(1000 + 10 * i)
        Ip, Fp = cases[partner][0](2000 + 10 * i)
        _say(f"[small] {name} (with {partner} on side 2)")
        with bf.Operation(name, partner) as op:
            O = op.run_kernel(0, I, F)
            Op_ = op.run_kernel(1, Ip, Fp)
        e = _check(name, O, oracle(I, F), tol, is_bf16)
        _check(partner, Op_, cases[partner][1](Ip, Fp), cases[partner][2], cases[partner][3])
        _say(f"[small] {name}: max rel err {e:.3e}")


@pytest.mark.parametrize("k1,k2,kind,suffix", FUSIONS)
def test_small_fusions_bit_exact(k1, k2, kind, suffix):
    cases = _cases()
    I1, F1 = cases[k1][0](77)
    I2, F2 = cases[k2][0](99)
    _say(f"[small-fuse] {k1} + {k2} {kind}{suffix}")
    with bf.Operation(k1, k2) as op:
        O1, O2 = op.run_kernel(0, I1, F1), op.run_kernel(1, I2, F2)
        fused = op.fused(kind, suffix)
        op.zero_outputs()
        Q1, Q2 = op.run_fuse(fused, I1, F1, I2, F2)
        # a second launch over the same buffers gives the same bytes (no state carried in LDS counters etc.)
        op.zero_outputs()
        R1, R2 = op.run_fuse(fused, I1, F1, I2, F2)
    for got, again, want, k in ((Q1, R1, O1, k1), (Q2, R2, O2, k2)):
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), f"{fused.name}: {k} differs from unfused"
        assert np.array_equal(again.view(np.uint8), want.view(np.uint8)), f"{fused.name}: {k} differs on relaunch"
    _check(k1, O1, cases[k1][1](I1, F1), cases[k1][2], cases[k1][3])
    _check(k2, O2, cases[k2][1](I2, F2), cases[k2][2], cases[k2][3])


def test_special_values():
    """Closed-form cases on the device: identity GEMM, constant LayerNorm row, RoPE at position 0,
    softmax of equal scores."""
    with bf.Operation("gemm_f32_64x32x48", "layernorm_8x256") as op:
        A = fill_uniform(5, 64 * 32, -1, 1).reshape(64, 32)
        B = np.zeros((32, 48), np.float32)
        B[np.arange(32), np.arange(32)] = 1.0
        C = op.run_kernel(0, A, B).reshape(64, 48)
        assert np.array_equal(C[:, :32], A) and np.all(C[:, 32:] == 0)
        x = np.full((8, 256), 3.25, np.float32)
        gb = np.concatenate([np.ones(256, np.float32), np.full(256, 0.5, np.float32)])
        assert np.array_equal(op.run_kernel(1, x, gb).ravel(), np.full(8 * 256, 0.5, np.float32))
    with bf.Operation("softmax_causal_2x256x256", "rmsnorm_rope_bf16_6x1024") as op:
        y = op.run_kernel(0, np.zeros((2, 256, 256), np.float32), np.zeros(1, np.float32)).reshape(2, 256, 256)
        for i in (0, 1, 7, 255):
            np.testing.assert_allclose(y[:, i, : i + 1], 1.0 / (i + 1), rtol=1e-6)
            assert np.all(y[:, i, i + 1:] == 0)
        x = f32_to_bf16(fill_normal(9, 6 * 1024, 0, 1))
        cosv, sinv = wl.rope_tables(6, 128, 500000.0)
        F = wl.pack_norm_rope_operand(f32_to_bf16(np.ones(1024, np.float32)), cosv, sinv)
        out = bf16_to_f32(op.run_kernel(1, x, F)).reshape(6, 1024)
        xf = bf16_to_f32(x).reshape(6, 1024).astype(np.float64)
        n0 = xf[0] / np.sqrt(np.mean(xf[0] ** 2) + 1e-5)            # position 0: rotation is the identity
        np.testing.assert_allclose(out[0], n0, rtol=1e-2, atol=1e-2 * np.sqrt(np.mean(n0 ** 2)))


def test_gelu_epilogue_over_the_whole_range():
    """tanh-GELU is evaluated as x / (1 + exp(-2u)) with the device's exp2 and reciprocal: check it
    from -60 to 60 (exp2 overflows to inf on one side and flushes to 0 on the other) through a
    selector GEMM, C[r, n] = gelu(B[k(r), n]), for each small GELU kernel."""
    for name, (M, K, N) in {"gemm_gelu_f32_64x192x288_d": (64, 192, 288), "gemm_gelu_f32_96x128x192": (96, 128, 192)}.items():
        rng = np.random.default_rng(7)
        k = rng.integers(0, K, M)
        A = np.zeros((M, K), np.float32)
        A[np.arange(M), k] = 1.0
        B = np.concatenate([np.linspace(-60.0, 60.0, K * N - 6), [0.0, -0.0, 1e-30, -1e-30, 88.0, -88.0]]).astype(np.float32)
        B = rng.permutation(B).reshape(K, N)
        x = B[k, :].astype(np.float64)
        want = 0.5 * x * (1.0 + np.tanh(0.797885 * (x + 0.044715 * x ** 3)))
        _say(f"[small] GELU range through {name}")
        with bf.Operation(name, "bias_relu_4096") as op:
            got = op.run_kernel(0, A.ravel(), B.ravel()).reshape(M, N).astype(np.float64)
        assert np.isfinite(got).all()
        err = np.abs(got - want) / np.maximum(np.abs(want), 1.0)
        assert err.max() <= 1e-5, f"{name}: max err {err.max():.3e} at x = {x.ravel()[err.argmax()]}"
