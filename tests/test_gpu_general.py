"""The operator ids of the reference's example configs (test-utils/examples/llm.yaml, resnet-18.yaml) that
the five benchmark configurations and tests/test_gpu_models.py do not reach: the Llama-3-8B dense layers
in fp32, bgemm_4 .. bgemm_17, and the ResNet-18 convolutions with other filter sizes, strides and image
sizes than 3x3 / 1 / 56.  Every kernel at full size against the CPU oracle (1e-5 of max(|ref|, rms)),
on selector inputs that make every output element one operand element exactly, and block-fused with a
LayerNorm, bit for bit against the two kernels launched back to back."""
import numpy as np
import pytest

import bfuse_project_amd as bf
from bfuse_project_amd.operation import fill_normal
from oracle import oracle as orf
from tests import oracle_cases

pytestmark = pytest.mark.gpu

PARTNER = "layernorm_512x768"


def _partner_inputs():
    x = fill_normal(0xF0, 512 * 768, 0.0, 1.0)
    gb = np.concatenate([fill_normal(0xF1, 768, 1.0, 0.1), fill_normal(0xF2, 768, 0.0, 0.1)])
    return x, gb


def _fused_equals_unfused(op, a, w, c):
    x, gb = _partner_inputs()
    y = op.run_kernel(1, x, gb)
    q1, q2 = op.run_fuse(op.fused("bfuse", "_c256"), a, w, x, gb)
    assert q1.tobytes() == c.tobytes() and q2.tobytes() == y.tobytes(), "fused output differs from the unfused kernels"


# ---- convolutions ---------------------------------------------------------------------------------
CONVS = [  # id, CI, H, W, CO, KH, KW, stride, padding
    ("conv2d_0", 3, 224, 224, 64, 7, 7, 2, 3), ("conv2d_2", 64, 56, 56, 64, 1, 1, 1, 0), ("conv2d_3", 64, 56, 56, 128, 3, 3, 2, 1),
    ("conv2d_5", 64, 56, 56, 128, 1, 1, 2, 0), ("conv2d_6", 128, 28, 28, 256, 3, 3, 2, 1), ("conv2d_7", 256, 14, 14, 256, 3, 3, 1, 1),
    ("conv2d_8", 128, 28, 28, 256, 1, 1, 2, 0), ("conv2d_9", 256, 14, 14, 512, 3, 3, 2, 1), ("conv2d_10", 512, 7, 7, 512, 3, 3, 1, 1),
    ("conv2d_11", 256, 14, 14, 512, 1, 1, 2, 0)]


@pytest.mark.parametrize("kid,ci,h,w,co,kh,kw,s,p", CONVS)
def test_resnet_convolution_against_the_oracle_on_selectors_and_fused(kid, ci, h, w, co, kh, kw, s, p):
    name = f"conv{kh}x{kw}s{s}p{p}_f32_{ci}x{h}x{w}_{co}"
    print(f"[general] {kid} -> {name}", flush=True)
    oh, ow = (h - kh + 2 * p) // s + 1, (w - kw + 2 * p) // s + 1
    xin = np.maximum(fill_normal(0xC00 + ci + h, ci * h * w, 0.0, 1.0), 0.0)
    wt = fill_normal(0xC80 + co + kh, co * ci * kh * kw, 0.0, 0.05)
    # selector filters: output channel c copies input channel (5c + 1) mod CI under tap (c mod KH, (2c + 1) mod KW),
    # so every output element is one (padded) input element exactly: a wrong tap offset, stride, padding,
    # channel group or pixel tail shows as a wrong element, not as a small error
    sel = np.zeros((co, ci, kh, kw), np.float32)
    cs = np.arange(co)
    sel[cs, (5 * cs + 1) % ci, cs % kh, (2 * cs + 1) % kw] = 1.0
    xsel = fill_normal(0xCF0 + len(kid) + co, ci * h * w, 0.0, 1.0)
    with bf.Operation(name, PARTNER) as op:
        assert tuple(op.k[0].shapes[2]) == (1, co, oh, ow)
        c = op.run_kernel(0, xin, wt)
        ysel = op.run_kernel(0, xsel, sel.ravel())
        _fused_equals_unfused(op, xin, wt, c)
        op.upload(0, xin, wt)
        t = float(np.mean(op.time("kernel1", warmup=10, reps=50)[0]))
    xp = np.pad(xsel.reshape(ci, h, w), ((0, 0), (p, p), (p, p)))
    want_sel = np.stack([xp[(5 * c_ + 1) % ci, c_ % kh:c_ % kh + s * oh:s, (2 * c_ + 1) % kw:(2 * c_ + 1) % kw + s * ow:s] for c_ in range(co)])
    assert np.array_equal(ysel.reshape(co, oh, ow), want_sel), "selector filters: an output element is not the input element it selects"
    want = orf.conv2d(xin.reshape(1, ci, h, w), wt.reshape(co, ci, kh, kw), s=s, p=p)
    st = oracle_cases.rel_stats(c, want, 1e-5)
    flops = 2.0 * co * ci * kh * kw * oh * ow
    print(f"[parity] {name}: worst |d|/max(|ref|,rms) {st['worst_floor_rel']:.3e}; {st['n_fail']} fail; {t:.1f} us "
          f"({flops / t * 1e-6:.1f} TFLOP/s)", flush=True)
    assert st["n_fail"] == 0


# ---- batched GEMMs --------------------------------------------------------------------------------
BGEMMS = [("bgemm_4", 16, 256, 64, 256), ("bgemm_5", 16, 256, 256, 64), ("bgemm_6", 16, 256, 80, 256), ("bgemm_7", 16, 256, 256, 80),
          ("bgemm_8", 16, 208, 64, 208), ("bgemm_9", 16, 208, 208, 64), ("bgemm_10", 16, 208, 80, 208), ("bgemm_11", 16, 208, 208, 80),
          ("bgemm_12", 1, 512, 64, 256), ("bgemm_13", 1, 512, 256, 64), ("bgemm_14", 1, 768, 64, 384), ("bgemm_15", 1, 768, 384, 64),
          ("bgemm_16", 1, 1024, 64, 512), ("bgemm_17", 1, 1024, 512, 64)]


@pytest.mark.parametrize("kid,b,m,k,n", BGEMMS)
def test_batched_gemm_against_the_oracle_on_selectors_and_fused(kid, b, m, k, n):
    """C[b] = A[b] . B[b]^T, B stored [b, N, K] (scripts/configure_kernels.py:14-19,40-48)."""
    name = f"bgemm_f32_{b}x{m}x{k}x{n}"
    print(f"[general] {kid} -> {name}", flush=True)
    a = fill_normal(0x1B0 + k + m, b * m * k, 0.0, 1.0)
    w = fill_normal(0x2B0 + n, b * n * k, 0.0, 0.125)
    with bf.Operation(name, PARTNER) as op:
        c = op.run_kernel(0, a, w)
        # A[b, r, :] = one-hot at k = (r + b) mod K  =>  C[b, r, j] = B[b, j, (r + b) mod K] exactly
        sel = np.zeros((b, m, k), np.float32)
        bi, ri = np.meshgrid(np.arange(b), np.arange(m), indexing="ij")
        sel[bi, ri, (ri + bi) % k] = 1.0
        cs = op.run_kernel(0, sel.ravel(), w)
        _fused_equals_unfused(op, a, w, c)
        op.upload(0, a, w)
        t = float(np.mean(op.time("kernel1", warmup=10, reps=50)[0]))
    W = w.reshape(b, n, k)
    want_sel = np.stack([W[i][:, (np.arange(m) + i) % k].T for i in range(b)])
    assert np.array_equal(cs.reshape(b, m, n), want_sel), "selector inputs: an output element is not the B element it selects"
    A = a.reshape(b, m, k)
    want = np.stack([orf.gemm_f32(A[i], W[i], b_is_nk=True) for i in range(b)])
    st = oracle_cases.rel_stats(c, want, 1e-5)
    print(f"[parity] {name}: worst |d|/max(|ref|,rms) {st['worst_floor_rel']:.3e}; {st['n_fail']} fail; {t:.1f} us "
          f"({2.0 * b * m * n * k / t * 1e-6:.1f} TFLOP/s)", flush=True)
    assert st["n_fail"] == 0


# ---- the Llama-3-8B dense layers in fp32, from a weight in the reference's (out, in) layout -------------
@pytest.mark.parametrize("kid,m,k,n", [("dense_4", 512, 4096, 4096), ("dense_6", 512, 4096, 14336), ("dense_7", 512, 14336, 4096)])
def test_llama_dense_layer_in_fp32_from_a_reference_layout_weight(kid, m, k, n):
    """The weight starts as the reference holds it, (out, in) = [N, K]; the library's transpose brings it to
    [K, N] once (checked byte for byte), the GEMM runs from that.  Every output against the oracle, selector
    inputs for every output element, and the fused kernel."""
    name = f"gemm_f32_{m}x{k}x{n}"
    print(f"[general] {kid} -> {name} (weight through transpose32_{n}x{k})", flush=True)
    a = fill_normal(0xA40 + k, m * k, 0.0, 1.0)
    w_nk = fill_normal(0xB40 + n, n * k, 0.0, 0.02)
    with bf.Operation(f"transpose32_{n}x{k}", "bias_relu_4096") as op:
        w_kn = op.run_kernel(0, w_nk, np.zeros(1, np.float32))
    assert np.array_equal(w_kn.reshape(k, n), w_nk.reshape(n, k).T)
    with bf.Operation(name, PARTNER) as op:
        c = op.run_kernel(0, a, w_kn)
        sel = np.zeros((m, k), np.float32)
        sel[np.arange(m), (np.arange(m) * 37) % k] = 1.0
        cs = op.run_kernel(0, sel.ravel(), w_kn)
        _fused_equals_unfused(op, a, w_kn, c)
        op.upload(0, a, w_kn)
        t = float(np.mean(op.time("kernel1", warmup=5, reps=20)[0]))
    W = w_nk.reshape(n, k)
    assert np.array_equal(cs.reshape(m, n), W[:, (np.arange(m) * 37) % k].T), "selector inputs: an output element is not the weight it selects"
    want = orf.gemm_f32(a.reshape(m, k), W, b_is_nk=True)            # every output element
    st = oracle_cases.rel_stats(c, want, 1e-5)
    print(f"[parity] {name}: all {m} x {n} outputs over K = {k}: worst |d|/max(|ref|,rms) {st['worst_floor_rel']:.3e}; "
          f"{st['n_fail']} fail; {t:.1f} us ({2.0 * m * n * k / t * 1e-6:.1f} TFLOP/s)", flush=True)
    assert st["n_fail"] == 0


@pytest.mark.parametrize("n,k", [(768, 768), (3072, 768), (768, 3072), (2304, 768), (1024, 4096), (512, 512)])
def test_weight_transposes_of_the_other_dense_layers(n, k):
    w_nk = fill_normal(0x7A0 + n + k, n * k, 0.0, 1.0)
    with bf.Operation(f"transpose32_{n}x{k}", "bias_relu_4096") as op:
        w_kn = op.run_kernel(0, w_nk, np.zeros(1, np.float32))
    assert np.array_equal(w_kn.reshape(k, n), w_nk.reshape(n, k).T)


def test_every_id_of_the_references_example_configs_runs_through_the_suite(tmp_path):
    """llm.yaml (26 ids) and resnet-18.yaml (12 ids) as the reference ships them: every id resolves (no
    --skip-missing), and a suite over a few of the new ids validates its fused kernels bit for bit."""
    import os
    import yaml
    from bfuse_project_amd import configure, suite
    ref = "/root/reference/test-utils/examples"
    cfg = tmp_path / "mixed.yaml"
    cfg.write_text(yaml.safe_dump({
        "FusionSet": [{"Set": ["bgemm_8", "conv2d_9", "conv2d_0"]}, {"Set": ["bgemm_11", "conv2d_10"]}],
        "KernelInfo": {"bgemm_8": [16, 208, 64, 208], "bgemm_11": [16, 208, 208, 80], "conv2d_9": [1, 14, 14, 512, 256, 3, 3, 2, 1],
                       "conv2d_0": [1, 224, 224, 64, 3, 7, 7, 2, 3], "conv2d_10": [1, 7, 7, 512, 512, 3, 3, 1, 1]}}))
    r = configure.configure(str(cfg), str(tmp_path / "o"))
    assert not r["missing"] and len(r["pairs"]) == 6
    rows = suite.run_suite(suite.load_info(str(tmp_path / "o" / "config" / "info.yaml")), str(tmp_path / "o"), validate=True, log=lambda m_: None)
    assert len(rows) == 6 and all(x["serial_ns"] > 0 and x["parallel_ns"] > 0 for x in rows)
    if os.path.isdir(ref):
        for name, count in (("llm.yaml", 26), ("resnet-18.yaml", 12)):
            with open(os.path.join(ref, name)) as f:
                doc = yaml.safe_load(f)
            ids = list(doc["KernelInfo"])
            doc["FusionSet"] = [{"Set": ids}, {"Set": ids}]
            p = tmp_path / name
            p.write_text(yaml.safe_dump(doc))
            r = configure.configure(str(p), str(tmp_path / ("o_" + name)))
            assert len(r["found"]) == count and not r["missing"]
