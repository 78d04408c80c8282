"""Pins for the oracle's pull-back of the Qwen3.5 attention input stage
(skyrl/tx/kernels/qwen3_5_qkv_lora.py:97-116, 148-164, 360-451): adjoint identities, automatic
differentiation in float64, and enumerated cases a wrong sign, a swapped half or a misplaced chunk
would break."""

import numpy as np
import pytest

from oracle import w8a8_oracle as o

F32 = np.float32
HALF_ULP = 2.0 ** -8


def test_rope_transpose_is_the_adjoint_and_the_inverse():
    rng = np.random.default_rng(3)
    rows, heads, d, rot, theta = 6, 3, 16, 8, 10000.0
    pos = np.asarray([0, 1, 7, 100, 4095, 33])
    x = o.bf16_round(rng.standard_normal((rows, heads, d)).astype(F32))
    y = o.bf16_round(rng.standard_normal((rows, heads, d)).astype(F32))
    rx = o.apply_partial_rope(x, pos, rot, theta).astype(np.float64)
    rty = o.apply_partial_rope_transpose(y, pos, rot, theta).astype(np.float64)
    # <R x, y> = <x, R^T y> up to the bf16 roundings of the two results
    lhs, rhs = np.sum(rx * y), np.sum(x * rty)
    assert abs(lhs - rhs) < 2e-2 * np.sqrt(np.sum(x.astype(np.float64) ** 2) * np.sum(y.astype(np.float64) ** 2)) / 10
    # a rotation: the transpose undoes it (one bf16 rounding per application)
    back = o.apply_partial_rope_transpose(o.apply_partial_rope(x, pos, rot, theta), pos, rot, theta)
    assert np.abs(back - x).max() <= 3 * HALF_ULP * np.abs(x).max()
    # position 0 and rotary_dim 0 leave the cotangent alone; the tail passes through at any position
    np.testing.assert_array_equal(o.apply_partial_rope_transpose(y[:1], np.asarray([0]), rot, theta), y[:1])
    np.testing.assert_array_equal(o.apply_partial_rope_transpose(y, pos, 0, theta), y)
    np.testing.assert_array_equal(rty[..., rot:], y[..., rot:])
    assert o.is_bf16_exact(rty.astype(F32))


def test_rope_transpose_signs_enumerated():
    # rot = 2: one pair (first, second) and the angle p / theta^0 = p
    pos = np.asarray([1])
    c = float(o.bf16_round(np.cos(np.asarray([1.0], F32)))[0])
    s = float(o.bf16_round(np.sin(np.asarray([1.0], F32)))[0])
    # [first cos + second sin, -first sin + second cos]
    got = o.apply_partial_rope_transpose(np.asarray([[[1.0, 0.0, 5.0]]], F32), pos, 2, 10000.0)
    np.testing.assert_array_equal(got[0, 0], [c, -s, 5.0])
    got = o.apply_partial_rope_transpose(np.asarray([[[0.0, 1.0, 5.0]]], F32), pos, 2, 10000.0)
    np.testing.assert_array_equal(got[0, 0], [s, c, 5.0])
    # and the forward rotation has the opposite sine signs
    fw = o.apply_partial_rope(np.asarray([[[1.0, 0.0, 5.0]]], F32), pos, 2, 10000.0)
    np.testing.assert_array_equal(fw[0, 0], [c, s, 5.0])


@pytest.mark.parametrize("eps", [1e-6, 0.25])
def test_delta_rms_norm_vjp_matches_automatic_differentiation(eps):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(17)
    x = o.bf16_round(rng.standard_normal((9, 24)).astype(F32) * 2.0)
    w = (0.3 * rng.standard_normal(24)).astype(F32)
    dy = o.bf16_round(rng.standard_normal((9, 24)).astype(F32))
    xt = torch.tensor(x.astype(np.float64), requires_grad=True)
    wt = torch.tensor(w.astype(np.float64), requires_grad=True)
    y = xt * torch.rsqrt((xt * xt).mean(-1, keepdim=True) + eps) * (1.0 + wt)
    y.backward(torch.tensor(dy.astype(np.float64)))
    dx, dw = o.delta_rms_norm_vjp(x, w, dy, eps)
    assert dx.shape == x.shape and o.is_bf16_exact(dx) and dw.shape == w.shape and dw.dtype == F32
    ref = xt.grad.numpy()
    scale = np.abs(dy * (1.0 + w)).max() / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + eps)
    assert np.all(np.abs(dx - ref) <= HALF_ULP * np.abs(ref) + 4e-6 * scale)
    np.testing.assert_allclose(dw, wt.grad.numpy(), rtol=2e-6, atol=2e-6)


def test_delta_rms_norm_vjp_closed_forms():
    # a cotangent with dy (1 + w) parallel to x is annihilated up to the eps term
    x = np.asarray([[1.0, -2.0, 4.0, 0.5]], dtype=F32)
    w = np.asarray([1.0, 0.0, 3.0, -0.5], dtype=F32)
    dy = (x / (1.0 + w)).astype(F32)
    dx, dw = o.delta_rms_norm_vjp(x, w, dy, 1e-12)
    assert np.abs(dx).max() < 1e-6
    inv = 1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2))
    np.testing.assert_allclose(dw, (dy * x * inv)[0], rtol=1e-6)
    # orthogonality: sum(x dx) vanishes as eps -> 0 (the norm is scale-free)
    rng = np.random.default_rng(8)
    x = o.bf16_round(rng.standard_normal((4, 32)).astype(F32))
    dy = o.bf16_round(rng.standard_normal((4, 32)).astype(F32))
    dx, _ = o.delta_rms_norm_vjp(x, np.zeros(32, F32), dy, 1e-12)
    assert np.abs(np.sum(x.astype(np.float64) * dx, axis=-1)).max() < 0.05
    # the weight cotangent sums over all rows: two copies of a row double it
    _, dw1 = o.delta_rms_norm_vjp(x[:1], w[:1].repeat(32), dy[:1], 1e-6)
    _, dw2 = o.delta_rms_norm_vjp(np.concatenate([x[:1], x[:1]]), w[:1].repeat(32), np.concatenate([dy[:1], dy[:1]]), 1e-6)
    np.testing.assert_allclose(dw2, 2.0 * dw1, rtol=1e-6)


CFG = dict(num_query_heads=4, num_kv_heads=2, head_dim=8, rotary_dim=4, rope_theta=10000.0, eps=1e-6)
WIDTH = 4 * 2 * 8 + 2 * 2 * 8


def test_reinterleave_is_the_adjoint_of_the_split():
    # with unit norm statistics out of the way (rotary_dim 0, weights 0) the K chunk still goes through
    # the norm, so the placement is checked on the pass-through outputs: gate and v
    rows = 2
    cfg = dict(CFG, rotary_dim=0)
    fused = o.bf16_round(np.random.default_rng(0).standard_normal((rows, WIDTH)).astype(F32))
    dq = np.zeros((rows, 4, 8), F32)
    dk = np.zeros((rows, 2, 8), F32)
    dv = np.arange(rows * 2 * 8, dtype=F32).reshape(rows, 2, 8) + 1.0
    dgate = -(np.arange(rows * 32, dtype=F32).reshape(rows, 32) + 1.0)
    dfused, dqw, dkw = o.qkv_split_norm_rope_bwd(fused, np.zeros(8, F32), np.zeros(8, F32), np.zeros(rows, np.int64),
                                                 dq, dk, dv, dgate, **cfg)
    assert dfused.shape == fused.shape and not dqw.any() and not dkw.any()
    # <split(f), (0, 0, dv, dgate)> = <f, dfused> for every f: compare against the forward's own split
    for probe in range(WIDTH):
        f = np.zeros((rows, WIDTH), F32)
        f[1, probe] = 1.0
        qpk = 2
        q_raw, k_raw, v_raw = o.split(f, (qpk * 2 * 8, 8, 8))
        gate = q_raw.reshape(rows, 4, 16)[..., 8:].reshape(rows, 32)
        want = np.sum(v_raw.reshape(rows, 2, 8) * dv) + np.sum(gate * dgate)
        assert dfused[1, probe] == want, probe
    # layout by hand: per kv head [q0 g0 q1 g1 k v], 8 wide each
    np.testing.assert_array_equal(dfused[0, 8:16], dgate[0, 0:8])
    np.testing.assert_array_equal(dfused[0, 24:32], dgate[0, 8:16])
    np.testing.assert_array_equal(dfused[0, 40:48], dv[0, 0])
    np.testing.assert_array_equal(dfused[0, 48 + 8:48 + 16], dgate[0, 16:24])
    np.testing.assert_array_equal(dfused[0, 48 + 40:48 + 48], dv[0, 1])
    assert not dfused[0, 0:8].any() and not dfused[0, 32:40].any()


def _stage_case(seed, m=10, k=32, n_ad=3, r=4):
    rng = np.random.default_rng(seed)
    hidden = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    w = o.quantize_frozen_weight((rng.standard_normal((k, WIDTH)) * 0.3).astype(F32), bits=8, group_size=k,
                                 scale_dtype="f32")
    a = o.bf16_round(rng.standard_normal((n_ad, k, r)).astype(F32) * 0.2)
    b = o.bf16_round(rng.standard_normal((n_ad, r, WIDTH)).astype(F32) * 0.2)
    s = rng.uniform(0.5, 2.0, n_ad).astype(F32)
    idx = rng.integers(0, n_ad, m)
    pos = rng.integers(0, 64, m)
    inw, qw, kw = (rng.standard_normal(n).astype(F32) * 0.2 for n in (k, 8, 8))
    dq = o.bf16_round(rng.standard_normal((m, 4, 8)).astype(F32))
    dk = o.bf16_round(rng.standard_normal((m, 2, 8)).astype(F32))
    dv = o.bf16_round(rng.standard_normal((m, 2, 8)).astype(F32))
    dgate = o.bf16_round(rng.standard_normal((m, 32)).astype(F32))
    return hidden, inw, qw, kw, w, a, b, s, idx, pos, dq, dk, dv, dgate


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_stage_backward_matches_automatic_differentiation(seed):
    """The whole rule against autograd through the smooth stage; the activation quantizer and the bf16
    casts between the stages bound the agreement (a few percent of each cotangent's norm)."""
    torch = pytest.importorskip("torch")
    hidden, inw, qw, kw, w, a, b, s, idx, pos, dq, dk, dv, dgate = _stage_case(seed)
    eps, d, rot, theta = CFG["eps"], 8, CFG["rotary_dim"], CFG["rope_theta"]
    t = lambda v: torch.tensor(np.asarray(v, dtype=np.float64), requires_grad=True)
    ht, inwt, qwt, kwt, at, bt, st = t(hidden), t(inw), t(qw), t(kw), t(a), t(b), t(s)
    it = torch.tensor(np.asarray(idx))

    def norm(x, wt):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + wt)

    def rope(x):  # [m, heads, d]
        half = rot // 2
        frac = 2.0 * torch.arange(half, dtype=torch.float64) / rot
        ang = torch.tensor(np.asarray(pos, dtype=np.float64))[:, None] / theta ** frac
        sin, cos = torch.sin(ang)[:, None, :], torch.cos(ang)[:, None, :]
        first, second = x[..., :half], x[..., half:rot]
        return torch.cat([first * cos - second * sin, first * sin + second * cos, x[..., rot:]], dim=-1)

    nrm = norm(ht, inwt)
    z = torch.einsum("mk,mkr->mr", nrm, at[it])
    fused = nrm @ torch.tensor(o.dequantize_frozen_weight(w).astype(np.float64)) \
        + torch.einsum("mr,mrn->mn", z, bt[it]) * st[it][:, None]
    m = hidden.shape[0]
    grouped = fused.reshape(m, 2, 6 * d)
    qg = grouped[..., :4 * d].reshape(m, 4, 2 * d)
    q = rope(norm(qg[..., :d], qwt))
    gate = qg[..., d:].reshape(m, 4 * d)
    kk = rope(norm(grouped[..., 4 * d:5 * d], kwt))
    v = grouped[..., 5 * d:]
    loss = (q * torch.tensor(dq.astype(np.float64))).sum() + (kk * torch.tensor(dk.astype(np.float64))).sum() \
        + (v * torch.tensor(dv.astype(np.float64))).sum() + (gate * torch.tensor(dgate.astype(np.float64))).sum()
    loss.backward()
    got = o.w8a8_qkv_lora_rope_bwd(hidden, inw, qw, kw, w, a, b, s, idx, pos, dq, dk, dv, dgate,
                                   relaxed_weight=False, **CFG)
    refs = {"dhidden": ht.grad, "d_input_norm_weight": inwt.grad, "d_q_norm_weight": qwt.grad,
            "d_k_norm_weight": kwt.grad, "d_lora_a": at.grad, "d_lora_b": bt.grad, "d_lora_scaling": st.grad}
    for name, ref in refs.items():
        ref = ref.numpy()
        err = np.linalg.norm(np.asarray(got[name], dtype=np.float64) - ref) / np.linalg.norm(ref)
        assert err < 0.04, (name, err)


def test_stage_backward_chains_and_vanishes():
    hidden, inw, qw, kw, w, a, b, s, idx, pos, dq, dk, dv, dgate = _stage_case(7)
    got = o.w8a8_qkv_lora_rope_bwd(hidden, inw, qw, kw, w, a, b, s, idx, pos, dq, dk, dv, dgate, **CFG)
    dfused, dqw, dkw = o.qkv_split_norm_rope_bwd(got["fused"], qw, kw, pos, dq, dk, dv, dgate, **CFG)
    np.testing.assert_array_equal(dfused, got["dfused"])
    np.testing.assert_array_equal(dqw, got["d_q_norm_weight"])
    dn, da, db, ds = o.quantized_lora_linear_multi_bwd(got["normalized"], w, a, b, s, idx, dfused, True)
    np.testing.assert_array_equal(dn, got["d_normalized"])
    dh, dinw = o.delta_rms_norm_vjp(hidden, inw, dn, CFG["eps"])
    np.testing.assert_array_equal(dh, got["dhidden"])
    np.testing.assert_array_equal(dinw, got["d_input_norm_weight"])
    zero = o.w8a8_qkv_lora_rope_bwd(hidden, inw, qw, kw, w, a, b, s, idx, pos, 0 * dq, 0 * dk, 0 * dv, 0 * dgate, **CFG)
    for name in ("dhidden", "d_input_norm_weight", "d_q_norm_weight", "d_k_norm_weight", "d_lora_a", "d_lora_b",
                 "d_lora_scaling", "dfused"):
        assert not np.asarray(zero[name]).any(), name
    # without adapters only the base term remains
    base = o.w8a8_qkv_lora_rope_bwd(hidden, inw, qw, kw, w, None, None, None, None, pos, dq, dk, dv, dgate, **CFG)
    assert base["d_lora_a"] is None and base["dhidden"].shape == hidden.shape
