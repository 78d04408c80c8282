"""Pins for the oracle's backward (quantized_lora.py:337-394): automatic differentiation of the
straight-through function in float64, finite differences, and identities a dropped term, a
transposed operand or a misplaced scaling would break."""

import numpy as np
import pytest

from oracle import w8a8_oracle as o

F32 = np.float32


def _case(seed, m=9, k=24, n=14, r=3, n_ad=1):
    rng = np.random.default_rng(seed)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    w = o.quantize_frozen_weight(rng.standard_normal((k, n)).astype(F32), bits=8, group_size=k, scale_dtype="f32")
    a = o.bf16_round(rng.standard_normal((n_ad, k, r)).astype(F32) * 0.3)
    b = o.bf16_round(rng.standard_normal((n_ad, r, n)).astype(F32) * 0.3)
    s = rng.uniform(0.5, 2.0, n_ad).astype(F32)
    dy = o.bf16_round(rng.standard_normal((m, n)).astype(F32))
    idx = rng.integers(0, n_ad, m)
    return x, w, a, b, s, dy, idx


def _autograd(x, w, a, b, s, dy, idx):
    torch = pytest.importorskip("torch")
    t = lambda v: torch.tensor(np.asarray(v, dtype=np.float64), requires_grad=True)
    xt, at, bt, st = t(x), t(a), t(b), t(s)
    wdeq = torch.tensor(o.dequantize_frozen_weight(w).astype(np.float64))
    it = torch.tensor(np.asarray(idx))
    z = torch.einsum("mk,mkr->mr", xt, at[it])
    low = torch.einsum("mr,mrn->mn", z, bt[it]) * st[it][:, None]
    y = xt @ wdeq + low           # straight-through base: the quantizers have no derivative
    y.backward(torch.tensor(np.asarray(dy, dtype=np.float64)))
    return [g.grad.numpy() for g in (xt, at, bt, st)]


@pytest.mark.parametrize("seed,n_ad", [(1, 1), (2, 1), (3, 4), (4, 5)])
def test_backward_matches_automatic_differentiation(seed, n_ad):
    x, w, a, b, s, dy, idx = _case(seed, n_ad=n_ad)
    want = _autograd(x, w, a, b, s, dy, idx)
    got = o.quantized_lora_linear_multi_bwd_f32(x, w, a, b, s, idx, dy)
    for g, ref, name in zip(got, want, ("dx", "dA", "dB", "ds")):
        np.testing.assert_allclose(g, ref, rtol=2e-6, atol=2e-5, err_msg=name)
    if n_ad == 1:
        dx1, da1, db1, ds1 = o.quantized_lora_linear_bwd_f32(x, w, a[0], b[0], s[0], dy)
        np.testing.assert_array_equal(dx1, got[0])
        np.testing.assert_array_equal(da1, got[1][0])
        np.testing.assert_array_equal(db1, got[2][0])
        assert ds1 == got[3][0]


def test_lora_cotangents_match_finite_differences():
    x, w, a, b, s, dy, _ = _case(7, m=5, k=8, n=6, r=2)
    a, b, s = a[0].astype(np.float64), b[0].astype(np.float64), float(s[0])
    loss = lambda a_, b_, s_: float(np.sum(dy.astype(np.float64) * ((x.astype(np.float64) @ a_) @ b_) * s_))
    _, da, db, ds = o.quantized_lora_linear_bwd_f32(x, w, a, b, s, dy)
    eps = 1e-4
    for (i, j) in [(0, 0), (3, 1), (7, 0)]:
        d = np.zeros_like(a); d[i, j] = eps
        assert abs((loss(a + d, b, s) - loss(a - d, b, s)) / (2 * eps) - da[i, j]) < 1e-3
    for (i, j) in [(0, 0), (1, 5), (0, 3)]:
        d = np.zeros_like(b); d[i, j] = eps
        assert abs((loss(a, b + d, s) - loss(a, b - d, s)) / (2 * eps) - db[i, j]) < 1e-3
    assert abs((loss(a, b, s + eps) - loss(a, b, s - eps)) / (2 * eps) - ds) < 1e-3


def test_backward_identities():
    x, w, a, b, s, dy, idx = _case(11, m=12, k=16, n=10, r=4, n_ad=3)
    dx, da, db, ds = o.quantized_lora_linear_multi_bwd_f32(x, w, a, b, s, idx, dy)
    wdeq = o.dequantize_frozen_weight(w)
    # B = 0: dx is the base pull-back alone, dA = 0, dscaling = 0, dB still sees x @ A
    dx0, da0, db0, ds0 = o.quantized_lora_linear_multi_bwd_f32(x, w, a, np.zeros_like(b), s, idx, dy)
    np.testing.assert_allclose(dx0, dy.astype(np.float64) @ wdeq.T.astype(np.float64), rtol=1e-6, atol=1e-5)
    assert not da0.any() and not ds0.any() and db0.any()
    # A = 0: dB = 0 and the LoRA part of dx vanishes, dA does not
    dx1, da1, db1, _ = o.quantized_lora_linear_multi_bwd_f32(x, w, np.zeros_like(a), b, s, idx, dy)
    np.testing.assert_array_equal(dx1, dx0)
    assert not db1.any() and da1.any()
    # an adapter without rows gets zeros; rows of other adapters do not leak into it
    idx2 = np.where(idx == 1, 0, idx)
    _, da2, db2, ds2 = o.quantized_lora_linear_multi_bwd_f32(x, w, a, b, s, idx2, dy)
    assert not da2[1].any() and not db2[1].any() and ds2[1] == 0
    # linear in dy
    dxh, dah, dbh, dsh = o.quantized_lora_linear_multi_bwd_f32(x, w, a, b, s, idx, dy * F32(0.5))
    np.testing.assert_allclose(dxh, dx * 0.5, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(dah, da * 0.5, rtol=1e-6, atol=1e-6)
    np.testing.assert_allclose(dsh, ds * 0.5, rtol=1e-6, atol=1e-6)
    # dscaling * s = <dB, B> = <dA, A> (Euler identities of the trilinear LoRA term)
    for g in range(3):
        lhs = float(ds[g]) * float(s[g])
        assert abs(lhs - float(np.sum(db[g].astype(np.float64) * b[g]))) < 1e-3 * max(1, abs(lhs))
        assert abs(lhs - float(np.sum(da[g].astype(np.float64) * a[g]))) < 1e-3 * max(1, abs(lhs))
    # the cast variant rounds each cotangent once
    cast = o.quantized_lora_linear_multi_bwd(x, w, a, b, s, idx, dy)
    np.testing.assert_array_equal(cast[0], o.bf16_round(dx))
    np.testing.assert_array_equal(cast[1], o.bf16_round(da))
    assert cast[3].dtype == F32


def test_relaxed_weight_policy_rounds_each_weight_once():
    """The ROCm pull-back contracts bf16(codes * scales) (rocm/w8a8_lora.py:326-330): dx moves by at
    most the rounding of the weights, the LoRA cotangents do not move at all."""
    x, w, a, b, s, dy, idx = _case(21, m=8, k=16, n=24, r=2, n_ad=2)
    exact = o.quantized_lora_linear_multi_bwd_f32(x, w, a, b, s, idx, dy)
    relaxed = o.quantized_lora_linear_multi_bwd_f32(x, w, a, b, s, idx, dy, relaxed_weight=True)
    wdeq = o.dequantize_frozen_weight(w)
    np.testing.assert_array_equal(o.pullback_weight(w, True), o.bf16_round(wdeq))
    np.testing.assert_array_equal(o.pullback_weight(w, False), wdeq)
    bound = np.abs(dy) @ np.abs(o.bf16_round(wdeq) - wdeq).T + 1e-5
    assert np.all(np.abs(relaxed[0] - exact[0]) <= bound) and np.any(relaxed[0] != exact[0])
    for i in (1, 2, 3):
        np.testing.assert_array_equal(relaxed[i], exact[i])
    base_only = o.quantized_lora_linear_multi_bwd_f32(x, w, a, np.zeros_like(b), s, idx, dy, relaxed_weight=True)[0]
    np.testing.assert_allclose(base_only, dy.astype(np.float64) @ o.bf16_round(wdeq).T.astype(np.float64),
                               rtol=1e-6, atol=1e-5)
