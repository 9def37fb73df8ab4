"""Pins the operator oracle (oracle/ops_ref.c) against PyTorch's CPU library routines in
float64 and against closed-form special cases.  The reference stores no operator outputs
(its only check is fused == unfused on one GPU), so these are the pins."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as orf

torch.set_num_threads(4)


def _rng(seed):
    return np.random.default_rng(seed)


def _close(a, b, rtol=2e-7, atol=1e-7):
    np.testing.assert_allclose(np.asarray(a, np.float64), np.asarray(b, np.float64), rtol=rtol, atol=atol)


@pytest.mark.parametrize("shape", [(7, 5, 3), (64, 48, 100), (33, 130, 257)])
@pytest.mark.parametrize("nk", [False, True])
def test_gemm_f32(shape, nk):
    M, N, K = shape
    r = _rng(1)
    A = r.uniform(-1, 1, (M, K)).astype(np.float32)
    B = r.uniform(-1, 1, (N, K) if nk else (K, N)).astype(np.float32)
    want = (torch.from_numpy(A).double() @ (torch.from_numpy(B).double().T if nk else torch.from_numpy(B).double())).float().numpy()
    got = orf.gemm_f32(A, B, b_is_nk=nk)
    assert np.array_equal(got, want) or np.max(np.abs(got - want)) <= 1e-6 * np.max(np.abs(want))
    # a transposed operand or a dropped k-term would fail this identity check
    I = np.eye(K, dtype=np.float32)
    if not nk:
        assert np.array_equal(orf.gemm_f32(A, I), A)


def test_gemm_gelu_epilogue():
    r = _rng(2)
    A = r.normal(0, 1, (40, 64)).astype(np.float32)
    B = r.normal(0, 0.3, (64, 24)).astype(np.float32)
    pre = orf.gemm_f32(A, B)
    got = orf.gemm_f32(A, B, epilogue=1)
    want = F.gelu(torch.from_numpy(pre).double(), approximate="tanh").numpy()
    # the dump's constant 0.797885 differs from sqrt(2/pi) in the 7th digit
    _close(got, want, rtol=5e-6, atol=5e-7)
    x = torch.from_numpy(pre).double()
    exact = (0.5 * x * (1 + torch.tanh(0.797885 * (x + 0.044715 * x ** 3)))).numpy()
    _close(got, exact, rtol=2e-7, atol=1e-9)


def test_gemm_bf16():
    r = _rng(3)
    A = orf.f32_to_bf16(r.normal(0, 1, (24, 96)).astype(np.float32))
    B = orf.f32_to_bf16(r.normal(0, 0.05, (96, 40)).astype(np.float32))
    got = orf.gemm_bf16(A, B)
    Ad, Bd = torch.from_numpy(orf.bf16_to_f32(A)).double(), torch.from_numpy(orf.bf16_to_f32(B)).double()
    want = (Ad @ Bd).float().bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    got_nk = orf.gemm_bf16(A, np.ascontiguousarray(B.T), b_is_nk=True)
    assert np.array_equal(got_nk, want)


def test_bf16_roundtrip_matches_torch():
    r = _rng(4)
    x = np.concatenate([r.normal(0, 1, 4096), [0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 1e-40, np.inf, -np.inf]]).astype(np.float32)
    got = orf.f32_to_bf16(x)
    want = torch.from_numpy(x).bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(orf.bf16_to_f32(got), torch.from_numpy(x).bfloat16().float().numpy())
    # ties go to even: 1 + 2^-8 is halfway between 1.0 and 1 + 2^-7 -> 1.0 ; 1 + 3*2^-8 -> 1 + 2^-6
    assert orf.bf16_to_f32(orf.f32_to_bf16(np.float32([1.00390625])))[0] == 1.0
    assert orf.bf16_to_f32(orf.f32_to_bf16(np.float32([1.01171875])))[0] == 1.015625


def test_bias_relu():
    r = _rng(5)
    x, b = r.normal(0, 1, 1000).astype(np.float32), r.normal(0, 0.1, 1000).astype(np.float32)
    assert np.array_equal(orf.bias_relu(x, b), np.maximum(x + b, 0))


def test_layernorm():
    r = _rng(6)
    x = r.normal(0.3, 2.0, (17, 768)).astype(np.float32)
    g, b = r.normal(1, 0.1, 768).astype(np.float32), r.normal(0, 0.1, 768).astype(np.float32)
    want = F.layer_norm(torch.from_numpy(x).double(), (768,), torch.from_numpy(g).double(), torch.from_numpy(b).double(), eps=1e-12).numpy()
    _close(orf.layernorm(x, g, b, 1e-12), want)
    # constant row -> beta (variance 0, eps keeps it finite)
    xc = np.full((2, 64), 3.25, np.float32)
    assert np.array_equal(orf.layernorm(xc, np.ones(64, np.float32), np.full(64, 0.5, np.float32), 1e-12), np.full((2, 64), 0.5, np.float32))
    # biased (1/d) variance: a +-1 row normalises to +-1 exactly
    xa = np.tile(np.float32([1, -1]), 8)[None]
    _close(orf.layernorm(xa, np.ones(16, np.float32), np.zeros(16, np.float32), 0.0), xa, rtol=0, atol=0)


def test_maxpool():
    r = _rng(7)
    x = r.normal(0, 1, (2, 3, 14, 11)).astype(np.float32)
    want = F.max_pool2d(torch.from_numpy(x), 3, 2, 1).numpy()
    assert np.array_equal(orf.maxpool2d(x), want)
    # monotone ramp: the maximum of each window is its bottom-right in-range element
    ramp = np.arange(8 * 8, dtype=np.float32).reshape(1, 1, 8, 8)
    y = orf.maxpool2d(ramp)
    assert y.shape == (1, 1, 4, 4)
    ih = np.minimum(np.arange(4) * 2 + 1, 7)
    assert np.array_equal(y[0, 0], ramp[0, 0][np.ix_(ih, ih)])
    # all-negative input: padding must not win
    assert np.all(orf.maxpool2d(-np.ones((1, 1, 6, 6), np.float32)) == -1)


def test_conv2d():
    r = _rng(8)
    x = np.maximum(r.normal(0, 1, (2, 5, 9, 7)), 0).astype(np.float32)
    w = r.normal(0, 0.05, (4, 5, 3, 3)).astype(np.float32)
    want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), padding=1).float().numpy()
    got = orf.conv2d(x, w)
    assert np.max(np.abs(got - want)) <= 1e-7
    want2 = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), stride=2, padding=1).float().numpy()
    assert np.max(np.abs(orf.conv2d(x, w, s=2, p=1) - want2)) <= 1e-7
    # a centre-tap delta kernel is the identity per channel (catches a flipped or shifted window)
    wd = np.zeros((5, 5, 3, 3), np.float32)
    for c in range(5):
        wd[c, c, 1, 1] = 1
    assert np.array_equal(orf.conv2d(x, wd), x)
    # an off-centre tap shifts the image (cross-correlation, not flipped convolution)
    ws = np.zeros((1, 5, 3, 3), np.float32); ws[0, 0, 0, 2] = 1
    y = orf.conv2d(x, ws)[0, 0]
    assert np.array_equal(y[1:, :-1], x[0, 0][:-1, 1:]) and np.all(y[0] == 0) and np.all(y[:, -1] == 0)


@pytest.mark.parametrize("ci,co,h,w,kh,kw,s,p", [(3, 8, 20, 18, 7, 7, 2, 3), (6, 4, 9, 9, 1, 1, 1, 0), (6, 4, 10, 8, 1, 1, 2, 0),
                                                 (5, 3, 14, 14, 3, 3, 2, 1), (4, 6, 7, 7, 3, 3, 1, 1), (2, 2, 11, 6, 5, 3, 3, 2)])
def test_conv2d_for_every_argument_list_of_the_resnet_layers(ci, co, h, w, kh, kw, s, p):
    """Filter sizes, strides and paddings of the reference's resnet-18.yaml (7x7 stride 2 padding 3; 1x1 with
    stride 1 and 2 and no padding; 3x3 stride 2; 3x3 on 7x7 images) and an asymmetric one, against the library
    routine, plus a closed form: a one-hot filter picks input pixels with the stride and the padding offset."""
    r = _rng(80 + kh * 10 + s)
    x = r.normal(0, 1, (1, ci, h, w)).astype(np.float32)
    wt = r.normal(0, 0.1, (co, ci, kh, kw)).astype(np.float32)
    want = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(wt).double(), stride=s, padding=p).float().numpy()
    got = orf.conv2d(x, wt, s=s, p=p)
    assert got.shape == want.shape == (1, co, (h - kh + 2 * p) // s + 1, (w - kw + 2 * p) // s + 1)
    assert np.max(np.abs(got - want)) <= 1e-6
    sel = np.zeros((1, ci, kh, kw), np.float32)
    a, b = kh - 1, kw // 2
    sel[0, ci - 1, a, b] = 1
    y = orf.conv2d(x, sel, s=s, p=p)[0, 0]
    xp = np.pad(x[0, ci - 1], p)
    oh, ow = y.shape
    assert np.array_equal(y, xp[a:a + s * oh:s, b:b + s * ow:s])


def test_softmax_causal():
    r = _rng(9)
    x = (r.normal(0, 1, (3, 33, 33)) / 8).astype(np.float32)
    mask = torch.triu(torch.full((33, 33), float("-inf"), dtype=torch.float64), 1)
    want = F.softmax(torch.from_numpy(x).double() + mask, dim=-1).numpy()
    got = orf.softmax_causal(x)
    _close(got, want)
    assert np.all(got[:, np.triu_indices(33, 1)[0], np.triu_indices(33, 1)[1]] == 0)
    _close(got.sum(-1), np.ones((3, 33)), rtol=0, atol=3e-7)
    assert np.all(got[:, 0, 0] == 1)
    # constant scores -> uniform over the visible prefix
    u = orf.softmax_causal(np.zeros((1, 8, 8), np.float32))[0]
    for i in range(8):
        _close(u[i, : i + 1], np.full(i + 1, 1 / (i + 1)), rtol=1e-7, atol=0)


def _hf_rope(t, cos, sin):
    half = t.shape[-1] // 2
    rot = torch.cat([-t[..., half:], t[..., :half]], -1)
    return t * cos + rot * sin


def test_rmsnorm_rope_bf16():
    r = _rng(10)
    S, heads, hd = 19, 4, 128
    x = orf.f32_to_bf16(r.normal(0, 1, (S, heads * hd)).astype(np.float32))
    w = orf.f32_to_bf16(r.normal(1, 0.1, heads * hd).astype(np.float32))
    cos, sin = orf.rope_tables(S, hd, 500000.0)
    # tables against the HF construction
    inv = 1.0 / (500000.0 ** (torch.arange(0, hd, 2, dtype=torch.float64) / hd))
    ang = torch.arange(S, dtype=torch.float64)[:, None] * inv[None]
    emb = torch.cat([ang, ang], -1)
    _close(cos, emb.cos().numpy(), rtol=0, atol=6e-8)
    _close(sin, emb.sin().numpy(), rtol=0, atol=6e-8)
    xd = torch.from_numpy(orf.bf16_to_f32(x)).double()
    wd = torch.from_numpy(orf.bf16_to_f32(w)).double()
    n = xd * torch.rsqrt(xd.pow(2).mean(-1, keepdim=True) + 1e-5)
    t = (wd * n).view(S, heads, hd)
    out = _hf_rope(t, torch.from_numpy(cos).double()[:, None], torch.from_numpy(sin).double()[:, None]).reshape(S, -1)
    want = out.float().bfloat16().view(torch.int16).numpy().view(np.uint16)
    got = orf.rmsnorm_rope_bf16(x, w, cos, sin, heads, 1e-5)
    # both round the same double value once; allow a 1-ulp flip on exact float32 double-rounding ties
    diff = np.abs(got.astype(np.int32) - want.astype(np.int32))
    assert diff.max() <= 1 and (diff > 0).mean() < 1e-3
    # position 0: cos=1, sin=0 -> RoPE is the identity, output is the RMSNorm alone
    want0 = (wd * n)[0].float().bfloat16().view(torch.int16).numpy().view(np.uint16)
    assert np.abs(got[0].astype(np.int32) - want0.astype(np.int32)).max() <= 1
    # rotation preserves the norm of each (j, j+64) pair
    g = orf.bf16_to_f32(got).reshape(S, heads, 2, hd // 2)
    tt = t.view(S, heads, 2, hd // 2).numpy()
    _close((g ** 2).sum(2), (tt ** 2).sum(2), rtol=2e-2, atol=1e-3)


def test_tolerance_counters():
    a = np.float32([1.0, 100.0, 1e-3, 0.0])
    o = a + np.float32([5e-6, 5e-4, 5e-6, 5e-6])
    assert orf.count_rel(o, a, 1e-5, floor_mag=1.0) == 0
    assert orf.count_rel(o, a, 1e-5, floor_mag=1e-6) == 2
    assert abs(orf.max_rel(o, a, 1.0) - 5e-6) < 1e-6
    assert np.isnan(orf.max_rel(np.float32([np.nan]), np.float32([1.0]), 1.0))
    assert orf.count_rel(np.float32([np.nan]), np.float32([1.0]), 1e-5, 1.0) == 1
