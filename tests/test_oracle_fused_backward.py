"""Pins for the oracle's pull-backs around the gate/up projection
(bf16_rms_gate_up_lora_swiglu_contiguous.py:541-574, 643-689): automatic differentiation in
float64, closed forms, and identities a dropped term, a wrong sign or swapped gate/up would break."""

import numpy as np
import pytest

from oracle import w8a8_oracle as o

F32 = np.float32
HALF_ULP = 2.0 ** -8  # bf16 round-to-nearest: relative error of one rounding


def _bf16_close(got, ref, extra=0.0):
    ref = np.asarray(ref, dtype=np.float64)
    bound = (HALF_ULP + extra) * np.abs(ref) + 1e-30 + extra * 1e-3
    bad = np.abs(np.asarray(got, dtype=np.float64) - ref) > bound
    assert not bad.any(), f"{int(bad.sum())} of {bad.size} beyond one bf16 rounding"


def test_swiglu_pullback_matches_automatic_differentiation():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(11)
    fused = o.bf16_round(rng.standard_normal((7, 24)).astype(F32) * 3.0)
    c = o.bf16_round(rng.standard_normal((7, 12)).astype(F32))
    ft = torch.tensor(fused.astype(np.float64), requires_grad=True)
    prod = torch.nn.functional.silu(ft[:, 0::2]) * ft[:, 1::2]
    prod.backward(torch.tensor(c.astype(np.float64)))
    got = o.swiglu_pullback_interleaved(fused, c)
    assert got.shape == fused.shape and o.is_bf16_exact(got)
    _bf16_close(got, ft.grad.numpy(), extra=2e-6)


def test_swiglu_pullback_closed_forms():
    # gate 0: sigmoid = 1/2, its derivative 1/4 is multiplied by the gate -> d_gate = c u / 2, d_up = 0
    fused = np.asarray([[0.0, 3.0, 0.0, -1.5]], dtype=F32)
    c = np.asarray([[2.0, 4.0]], dtype=F32)
    np.testing.assert_array_equal(o.swiglu_pullback_interleaved(fused, c), [[3.0, 0.0, -3.0, 0.0]])
    # saturated gate: silu is the identity, d_up = c g, d_gate = c u; far negative: everything vanishes
    fused = np.asarray([[40.0, 0.5, -100.0, 7.0]], dtype=F32)
    got = o.swiglu_pullback_interleaved(fused, np.asarray([[0.25, 3.0]], dtype=F32))
    np.testing.assert_array_equal(got, [[0.125, 10.0, 0.0, 0.0]])
    assert np.isfinite(o.swiglu_pullback_interleaved(np.asarray([[-3e38, 1.0]], F32), np.ones((1, 1), F32))).all()
    # gate and up are the even and the odd columns: swapping them changes the answer
    a = o.swiglu_pullback_interleaved(np.asarray([[1.0, 2.0]], F32), np.ones((1, 1), F32))
    b = o.swiglu_pullback_interleaved(np.asarray([[2.0, 1.0]], F32), np.ones((1, 1), F32))
    assert a[0, 1] == o.bf16_round(o.silu(np.asarray([1.0], F32)))[0]
    assert b[0, 1] == o.bf16_round(o.silu(np.asarray([2.0], F32)))[0]


def test_swiglu_pullback_is_linear_in_the_cotangent():
    rng = np.random.default_rng(5)
    fused = o.bf16_round(rng.standard_normal((3, 16)).astype(F32))
    c = o.bf16_round(rng.standard_normal((3, 8)).astype(F32))
    np.testing.assert_array_equal(o.swiglu_pullback_interleaved(fused, 4.0 * c),
                                  4.0 * o.swiglu_pullback_interleaved(fused, c))
    np.testing.assert_array_equal(o.swiglu_pullback_interleaved(fused, np.zeros_like(c)), np.zeros_like(fused))


@pytest.mark.parametrize("eps", [1e-6, 0.5])
def test_rms_norm_pullback_matches_automatic_differentiation(eps):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(21)
    x = o.bf16_round(rng.standard_normal((6, 40)).astype(F32) * 2.0)
    gamma = (1.0 + 0.3 * rng.standard_normal(40)).astype(F32)
    dn = o.bf16_round(rng.standard_normal((6, 40)).astype(F32))
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    n = xt * torch.rsqrt((xt * xt).mean(-1, keepdim=True) + eps) * torch.tensor(gamma.astype(np.float64))
    n.backward(torch.tensor(dn.astype(np.float64)))
    got = o.rms_norm_pullback(x, gamma, dn, eps)
    assert got.shape == x.shape and o.is_bf16_exact(got)
    ref = xt.grad.numpy()
    # cancellation between the two terms: bound the error by the size of the terms, not of the result
    scale = np.abs(dn * gamma).max() / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps)
    assert np.abs(got - ref).max() <= (HALF_ULP * np.abs(ref) + 4e-6 * scale).max()
    assert np.all(np.abs(got - ref) <= HALF_ULP * np.abs(ref) + 4e-6 * scale)


def test_rms_norm_pullback_closed_forms():
    # a cotangent along x (dn * gamma = alpha x) is annihilated up to the eps term: the norm is scale-free
    rng = np.random.default_rng(3)
    x = o.bf16_round(rng.standard_normal((4, 64)).astype(F32) + 3.0)
    gamma = np.full(64, 2.0, dtype=F32)
    dn = (0.5 * x).astype(F32)   # p = x exactly
    dx = o.rms_norm_pullback(x, gamma, dn, 1e-12)
    assert np.abs(dx).max() <= 1e-6 * np.abs(x).max()
    # one-element rows: n = x / sqrt(x^2 + eps) gamma, dn/dx = gamma eps / (x^2 + eps)^(3/2)
    x1 = np.asarray([[2.0], [-0.5]], dtype=F32)
    eps = 0.25
    want = 3.0 * 1.5 * eps / (x1.astype(np.float64) ** 2 + eps) ** 1.5
    got = o.rms_norm_pullback(x1, np.asarray([1.5], F32), np.full((2, 1), 3.0, F32), eps)
    np.testing.assert_allclose(got, want, rtol=2 * HALF_ULP)
    # orthogonality: sum_k x dx = (sum_k x p) inv eps / den
    x = o.bf16_round(rng.standard_normal((5, 32)).astype(F32))
    gamma = (1.0 + 0.1 * rng.standard_normal(32)).astype(F32)
    dn = o.bf16_round(rng.standard_normal((5, 32)).astype(F32))
    eps = 0.125
    dx = o.rms_norm_pullback(x, gamma, dn, eps).astype(np.float64)
    den = (x.astype(np.float64) ** 2).mean(-1) + eps
    ic = (x.astype(np.float64) * (dn * gamma)).sum(-1)
    np.testing.assert_allclose((x * dx).sum(-1), ic * eps / den ** 1.5, atol=0.05)
    # zero cotangent, and a zero row (inv = 1 / sqrt(eps), no NaN)
    np.testing.assert_array_equal(o.rms_norm_pullback(x, gamma, np.zeros_like(dn), eps), np.zeros_like(x))
    z = o.rms_norm_pullback(np.zeros((1, 8), F32), np.ones(8, F32), np.ones((1, 8), F32), 1e-6)
    np.testing.assert_allclose(z, np.full((1, 8), 1000.0), rtol=HALF_ULP)


def _fused_case(seed, m=12, k=48, n=32, r=4, n_ad=3):
    rng = np.random.default_rng(seed)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32) * 1.5)
    gamma = (1.0 + 0.2 * rng.standard_normal(k)).astype(F32)
    w = o.quantize_frozen_weight(rng.standard_normal((k, n)).astype(F32) * 0.2, bits=8, group_size=k,
                                 scale_dtype="f32")
    a = o.bf16_round(rng.standard_normal((n_ad, k, r)).astype(F32) * 0.2)
    b = o.bf16_round(rng.standard_normal((n_ad, r, n)).astype(F32) * 0.2)
    s = rng.uniform(0.5, 2.0, n_ad).astype(F32)
    idx = rng.integers(0, n_ad, m)
    c = o.bf16_round(rng.standard_normal((m, n // 2)).astype(F32))
    return x, gamma, w, a, b, s, idx, c


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_fused_backward_matches_automatic_differentiation(seed):
    """The whole rule against autograd through the smooth function; the activation quantizer and the
    bf16 casts between the stages bound the agreement (a few percent of each cotangent's norm)."""
    torch = pytest.importorskip("torch")
    x, gamma, w, a, b, s, idx, c = _fused_case(seed)
    eps = 1e-6
    t = lambda v: torch.tensor(np.asarray(v, dtype=np.float64), requires_grad=True)
    xt, at, bt, st = t(x), t(a), t(b), t(s)
    it = torch.tensor(np.asarray(idx))
    nrm = xt * torch.rsqrt((xt * xt).mean(-1, keepdim=True) + eps) * torch.tensor(gamma.astype(np.float64))
    z = torch.einsum("mk,mkr->mr", nrm, at[it])
    low = torch.einsum("mr,mrn->mn", z, bt[it]) * st[it][:, None]
    fused = nrm @ torch.tensor(o.dequantize_frozen_weight(w).astype(np.float64)) + low
    prod = torch.nn.functional.silu(fused[:, 0::2]) * fused[:, 1::2]
    prod.backward(torch.tensor(c.astype(np.float64)))
    got = o.w8a8_rms_gate_up_lora_swiglu_bwd(x, gamma, w, a, b, s, idx, c, eps, relaxed_weight=False)
    for g, ref, name in zip(got, (xt.grad, at.grad, bt.grad, st.grad), ("dx", "dA", "dB", "ds")):
        ref = ref.numpy()
        err = np.linalg.norm(np.asarray(g, dtype=np.float64) - ref) / np.linalg.norm(ref)
        assert err < 0.04, (name, err)


def test_fused_backward_stages_chain():
    x, gamma, w, a, b, s, idx, c = _fused_case(9)
    (dx, da, db, ds), st = o.w8a8_rms_gate_up_lora_swiglu_bwd(x, gamma, w, a, b, s, idx, c, return_stages=True)
    np.testing.assert_array_equal(st["d_fused"], o.swiglu_pullback_interleaved(st["fused"], c))
    dn, da2, db2, ds2 = o.quantized_lora_linear_multi_bwd(st["normalized"], w, a, b, s, idx, st["d_fused"], True)
    np.testing.assert_array_equal(dn, st["d_normalized"])
    np.testing.assert_array_equal(dx, o.rms_norm_pullback(x, gamma, dn))
    np.testing.assert_array_equal(da, da2)
    np.testing.assert_array_equal(db, db2)
    np.testing.assert_array_equal(ds, ds2)
    # a zero cotangent gives zero everywhere
    zero = o.w8a8_rms_gate_up_lora_swiglu_bwd(x, gamma, w, a, b, s, idx, np.zeros_like(c))
    for g in zero:
        assert not np.asarray(g).any()
