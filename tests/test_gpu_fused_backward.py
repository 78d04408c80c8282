"""GPU parity of the fused RMSNorm -> gate/up + LoRA -> SwiGLU backward (through the C ABI).

The two memory-bound pull-backs are compared with the CPU oracle on the same inputs to
|a - b| <= 2e-2 + 1e-2 |b| (float32 arithmetic in the reference's order; exp, reciprocal and the
row sums differ in their last bits).  The whole rule is checked stage by stage on the device's own
intermediates with that tolerance, and end to end against the oracle with the reference's W8A8
gate (relative L2 < 1e-2, cosine >= 0.9999).
"""

import numpy as np
import pytest

from oracle import w8a8_oracle as o
import w8a8_cases as wc

pytestmark = pytest.mark.gpu
F32 = np.float32


@pytest.fixture(scope="module")
def dev():
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def pkg():
    from __graft_entry__ import load_package

    p = load_package()
    p._native.load()
    return p


def _t(dev, v, dt=None):
    import torch

    if v is None:
        return None
    return torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(dt or torch.bfloat16)


def _np(v):
    import torch

    return v.detach().to(torch.float32).cpu().numpy()


@pytest.mark.parametrize("m,n,scale", [(1, 8, 1.0), (37, 264, 3.0), (256, 4096, 1.0), (5, 24, 30.0)])
def test_swiglu_backward_matches_oracle(dev, pkg, m, n, scale):
    import torch

    rng = np.random.default_rng(m * 131 + n)
    fused = o.bf16_round(rng.standard_normal((m, n)).astype(F32) * scale)
    c = o.bf16_round(rng.standard_normal((m, n // 2)).astype(F32))
    print(f"[case] swiglu backward m={m} n={n}", flush=True)
    want = o.swiglu_pullback_interleaved(fused, c)
    ft, ct = _t(dev, fused), _t(dev, c)
    got = pkg.w8a8_lora.swiglu_backward(ft, ct)
    torch.cuda.synchronize()
    rep = wc.compare(_np(got), want)
    print(f"[fused backward parity] swiglu m{m}n{n} {rep}", flush=True)
    assert rep["violations"] == 0, rep
    assert torch.equal(ft, _t(dev, fused))          # the input is untouched ...
    same = pkg.w8a8_lora.swiglu_backward(ft, ct, in_place=True)
    torch.cuda.synchronize()
    assert same.data_ptr() == ft.data_ptr() and torch.equal(same, got)   # ... unless asked for


@pytest.mark.parametrize("m,k,eps", [(1, 8, 1e-6), (19, 1000, 1e-6), (64, 4096, 1e-5), (7, 37, 1e-6), (3, 12288, 1e-6)])
def test_rms_norm_backward_matches_oracle(dev, pkg, m, k, eps):
    import torch

    rng = np.random.default_rng(m * 7 + k)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32) * 2.0)
    gamma = (1.0 + 0.2 * rng.standard_normal(k)).astype(F32)
    dn = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    print(f"[case] rms norm backward m={m} k={k}", flush=True)
    want = o.rms_norm_pullback(x, gamma, dn, eps)
    xt, gt, dt = _t(dev, x), _t(dev, gamma, torch.float32), _t(dev, dn)
    got = pkg.w8a8_lora.rms_norm_backward(xt, gt, dt, eps=eps)
    torch.cuda.synchronize()
    rep = wc.compare(_np(got), want)
    print(f"[fused backward parity] rms m{m}k{k} {rep}", flush=True)
    assert rep["violations"] == 0, rep
    assert rep["bitwise_fraction"] > 0.98, rep
    same = pkg.w8a8_lora.rms_norm_backward(xt, gt, dt, eps=eps, in_place=True)
    torch.cuda.synchronize()
    assert same.data_ptr() == dt.data_ptr() and torch.equal(same, got)


def _fused_case(seed, m, k, n, r, n_ad):
    rng = np.random.default_rng(seed)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32) * 1.5)
    delta = (0.2 * rng.standard_normal(k)).astype(F32)
    codes = rng.integers(-127, 128, (k, n)).astype(np.int8)
    sw = rng.uniform(0.2, 1.0, (1, n)).astype(F32) / (127.0 * np.sqrt(k))
    w = o.GroupQuantizedWeight(codes=codes, scales=sw.astype(F32), original_in_features=k, padded_in_features=k,
                               bits=8, group_size=k)
    a = o.bf16_round(rng.standard_normal((n_ad, k, r)).astype(F32) * 0.05)
    b = o.bf16_round(rng.standard_normal((n_ad, r, n)).astype(F32) * 0.05)
    s = rng.uniform(0.5, 2.0, n_ad).astype(F32)
    idx = rng.integers(0, n_ad, m).astype(np.int32)
    c = o.bf16_round(rng.standard_normal((m, n // 2)).astype(F32))
    return x, delta, w, a, b, s, idx, c


FUSED_CASES = [
    # m, k, n, r, adapters
    (8, 256, 512, 8, 2),        # recomputed by the skinny-M forward
    (70, 384, 776, 16, 3),      # ragged rows and columns
    (300, 1024, 2048, 32, 4),   # several row tiles
    (129, 200, 264, 5, 1),      # K % 8 == 0 but not a tile multiple, one adapter
]


@pytest.mark.parametrize("m,k,n,r,n_ad", FUSED_CASES)
def test_fused_backward_through_autograd(dev, pkg, m, k, n, r, n_ad):
    import torch

    x, delta, w, a, b, s, idx, c = _fused_case(m + k + n, m, k, n, r, n_ad)
    gamma = (F32(1.0) + delta).astype(F32)
    eps = 1e-6
    print(f"[case] fused backward m={m} k={k} n={n} r={r} adapters={n_ad}", flush=True)
    ql, w8 = pkg.quantized_lora, pkg.w8a8_lora
    wt = ql.GroupQuantizedWeight(torch.from_numpy(w.codes).to(dev), torch.from_numpy(w.scales).to(dev), k, k, 8, k)
    xt = _t(dev, x).requires_grad_(True)
    at = _t(dev, a).requires_grad_(True)
    bt = _t(dev, b).requires_grad_(True)
    st = _t(dev, s, torch.float32).requires_grad_(True)
    it = _t(dev, idx, torch.int32)
    dlt = _t(dev, delta, torch.float32).requires_grad_(True)
    out = w8.w8a8_rms_gate_up_lora_swiglu(xt, dlt, wt, at, bt, st, enabled=True, eps=eps, rms_is_delta=True,
                                          adapter_indices=it)
    assert out.requires_grad and tuple(out.shape) == (m, n // 2)
    want_out, stages = o.w8a8_rms_gate_up_lora_swiglu(x, gamma, w, a, b, s, idx, eps, return_stages=True)
    rep = wc.compare(_np(out), want_out)
    assert rep["violations"] == 0, rep
    out.backward(_t(dev, c))
    torch.cuda.synchronize()
    assert dlt.grad is None                       # the norm weight is a constant of the rule
    got = [_np(g.grad) for g in (xt, at, bt, st)]
    # end to end against the oracle
    want = o.w8a8_rms_gate_up_lora_swiglu_bwd(x, gamma, w, a, b, s, idx, c, eps)
    for g, ref, name in zip(got[:3], want[:3], ("dx", "dA", "dB")):
        gate = o.numerical_gate(g, ref)
        print(f"[fused backward parity] m{m}k{k}n{n} {name} {gate}", flush=True)
        assert gate["relative_l2"] < 1e-2 and gate["cosine"] >= 0.9999, (name, gate)
    np.testing.assert_allclose(got[3], want[3], rtol=1e-2, atol=1e-2)
    # stage by stage on the device's own intermediates
    fused_dev, aux = w8.forward(_t(dev, x), wt, _t(dev, a), _t(dev, b), _t(dev, s, torch.float32),
                                adapter_indices=it, rms_gamma=_t(dev, gamma, torch.float32), eps=eps, return_aux=True)
    fused_np, norm_np = _np(fused_dev), _np(aux["normalized"])
    np.testing.assert_array_equal(norm_np, stages["normalized"])
    d_fused = _np(w8.swiglu_backward(fused_dev, _t(dev, c)))
    rep = wc.compare(d_fused, o.swiglu_pullback_interleaved(fused_np, c))
    assert rep["violations"] == 0, rep
    dn_dev, da_dev, db_dev, ds_dev = w8.backward(aux["normalized"], _t(dev, d_fused), wt, _t(dev, a), _t(dev, b),
                                                 _t(dev, s, torch.float32), adapter_indices=it)
    ref_mid = o.quantized_lora_linear_multi_bwd(norm_np, w, a, b, s, idx, d_fused, relaxed_weight=True)
    for g, ref, name in zip((dn_dev, da_dev, db_dev), ref_mid[:3], ("dn", "dA", "dB")):
        rep = wc.compare(_np(g), ref)
        assert rep["violations"] == 0, (name, rep)
    np.testing.assert_array_equal(_np(da_dev), got[1])   # the rule is exactly this chain
    np.testing.assert_array_equal(_np(db_dev), got[2])
    dx_dev = w8.rms_norm_backward(_t(dev, x), _t(dev, gamma, torch.float32), dn_dev, eps=eps)
    rep = wc.compare(_np(dx_dev), o.rms_norm_pullback(x, gamma, _np(dn_dev), eps))
    assert rep["violations"] == 0, rep
    np.testing.assert_array_equal(_np(dx_dev), got[0])


def test_same_named_entry_point_is_differentiable(dev, pkg):
    import torch

    m, k, n, r = 40, 256, 512, 8
    x, delta, w, a, b, s, idx, c = _fused_case(77, m, k, n, r, 1)
    ql = pkg.quantized_lora
    fn = pkg.bf16_rms_gate_up_lora_swiglu_contiguous.bf16_rms_gate_up_lora_swiglu_contiguous
    wt = ql.GroupQuantizedWeight(torch.from_numpy(w.codes).to(dev), torch.from_numpy(w.scales).to(dev), k, k, 8, k)
    xt = _t(dev, x).reshape(2, 20, k).requires_grad_(True)
    at = _t(dev, a[0]).requires_grad_(True)
    bt = _t(dev, b[0]).requires_grad_(True)
    out = fn(xt, _t(dev, delta), wt, at, bt, torch.tensor(float(s[0]), device=dev), enabled=True)
    assert tuple(out.shape) == (2, 20, n // 2)
    out.backward(_t(dev, c).reshape(2, 20, n // 2))
    torch.cuda.synchronize()
    want = o.w8a8_rms_gate_up_lora_swiglu_bwd(x, (F32(1.0) + delta).astype(F32), w, a, b, s, np.zeros(m, np.int32), c)
    for g, ref, name in zip((xt.grad.reshape(m, k), at.grad, bt.grad), (want[0], want[1][0], want[2][0]),
                            ("dx", "dA", "dB")):
        gate = o.numerical_gate(_np(g), ref)
        assert gate["relative_l2"] < 1e-2 and gate["cosine"] >= 0.9999, (name, gate)
    # without gradients the forward alone runs
    with torch.no_grad():
        plain = fn(xt, _t(dev, delta), wt, at, bt, torch.tensor(float(s[0]), device=dev), enabled=True)
    assert not plain.requires_grad and torch.equal(plain, out.detach())


def test_fused_backward_rejects_bad_arguments(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    f = torch.zeros(4, 16, dtype=torch.bfloat16, device=dev)
    c = torch.zeros(4, 8, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        w8.swiglu_backward(f[:, :12], c[:, :6])             # N % 8
    with pytest.raises(ValueError):
        w8.swiglu_backward(f, c[:, :4])
    with pytest.raises(TypeError):
        w8.swiglu_backward(f.float(), c)
    g = torch.ones(16, dtype=torch.float32, device=dev)
    with pytest.raises(ValueError):
        w8.rms_norm_backward(f, g[:8], f)
    with pytest.raises(ValueError):
        w8.rms_norm_backward(f, g, f[:2])
    with pytest.raises(ValueError):
        w8.rms_norm_backward(f, g, f, eps=0.0)
    with pytest.raises(TypeError):
        w8.rms_norm_backward(f.float(), g, f)
    lib = pkg._native.load()
    st = lib.mi355_w8a8_swiglu_bwd_v1(f.data_ptr(), c.data_ptr(), f.data_ptr() + 16, 2, 16, None)
    assert pkg._native.STATUS[st] == "ERR_ALIAS"
    st = lib.mi355_w8a8_rms_norm_bwd_v1(f.data_ptr(), g.data_ptr(), f.data_ptr(), f.data_ptr(), 4, 16, 1e-6, None)
    assert pkg._native.STATUS[st] == "ERR_ALIAS"            # dx over x
    st = lib.mi355_w8a8_rms_norm_bwd_v1(None, g.data_ptr(), f.data_ptr(), f.data_ptr(), 4, 16, 1e-6, None)
    assert pkg._native.STATUS[st] == "ERR_NULL"


def test_fused_backward_full_size_properties(dev, pkg):
    """Qwen3-8B gate/up at M = 4096: the stages against float32 torch formulas, exact linearity in
    the cotangent (powers of two pass through every stage unchanged), zero in -> zero out."""
    import torch

    torch.manual_seed(5)
    m, k, n, r, n_ad = 4096, 4096, 24576, 32, 8
    print(f"[case] fused backward full size m={m} k={k} n={n}", flush=True)
    ql, w8 = pkg.quantized_lora, pkg.w8a8_lora
    codes = torch.randint(-127, 128, (k, n), dtype=torch.int8, device=dev)
    scales = (torch.rand(1, n, device=dev) * 0.8 + 0.2) / (127.0 * k ** 0.5)
    wt = w8.prepare_weight(ql.GroupQuantizedWeight(codes, scales, k, k, 8, k))
    x = (torch.randn(m, k, device=dev) * 1.5).to(torch.bfloat16)
    gamma = 1.0 + 0.2 * torch.randn(k, device=dev)
    a = (torch.randn(n_ad, k, r, device=dev) * 0.05).to(torch.bfloat16)
    b = (torch.randn(n_ad, r, n, device=dev) * 0.05).to(torch.bfloat16)
    s = torch.rand(n_ad, device=dev) + 0.5
    idx = torch.randint(0, n_ad, (m,), dtype=torch.int32, device=dev)
    c = torch.randn(m, n // 2, device=dev).to(torch.bfloat16)

    fused = w8.forward(x, wt, a, b, s, adapter_indices=idx, rms_gamma=gamma)
    d_fused = w8.swiglu_backward(fused, c)
    g32, u32, c32 = fused[:, 0::2].float(), fused[:, 1::2].float(), c.float()
    sig = torch.sigmoid(g32)
    ref = torch.stack(((c32 * u32) * sig + (g32 * (c32 * u32)) * (sig * (1 - sig)), c32 * (g32 * sig)), dim=-1)
    ref = ref.reshape(m, n).to(torch.bfloat16)
    bad = (d_fused.float() - ref.float()).abs() > 2e-2 + 1e-2 * ref.float().abs()
    assert int(bad.sum()) == 0
    del g32, u32, c32, sig, bad

    dn = torch.randn(m, k, device=dev).to(torch.bfloat16)
    dx = w8.rms_norm_backward(x, gamma, dn)
    x32, p = x.float(), dn.float() * gamma
    den = (x32.double() ** 2).mean(-1, keepdim=True).float() + 1e-6
    inv = 1.0 / den.sqrt()
    t = ((x32.double() * p.double()).sum(-1, keepdim=True).float() * (-0.5 * (inv / den))) / k
    ref = ((p * inv + x32 * t) + t * x32).to(torch.bfloat16)
    assert float((dx.float() - ref.float()).abs().max()) <= 2e-2
    assert float((dx != ref).float().mean()) < 0.01

    one = w8.rms_gate_up_swiglu_backward(x, gamma, wt, a, b, s, c, adapter_indices=idx)
    two = w8.rms_gate_up_swiglu_backward(x, gamma, wt, a, b, s, c * 2, adapter_indices=idx)
    zero = w8.rms_gate_up_swiglu_backward(x, gamma, wt, a, b, s, torch.zeros_like(c), adapter_indices=idx)
    torch.cuda.synchronize()
    for g1, g2, g0 in zip(one, two, zero):
        assert torch.isfinite(g1.float()).all()
        assert torch.equal(g2.float(), g1.float() * 2)
        assert not g0.any()
    assert float(one[0].float().abs().mean()) > 0


def test_saved_projection_and_recomputation_agree(dev, pkg):
    """The training forward that keeps the projection (the reference's choice) and the one that keeps
    nothing give bit-identical outputs and cotangents; the stand-alone SwiGLU kernel reproduces the
    fused epilogue bit for bit."""
    import torch

    m, k, n, r, n_ad = 150, 512, 1032, 16, 3
    x, delta, w, a, b, s, idx, c = _fused_case(31, m, k, n, r, n_ad)
    gamma = _t(dev, (F32(1.0) + delta).astype(F32), torch.float32)
    ql, w8 = pkg.quantized_lora, pkg.w8a8_lora
    wt = ql.GroupQuantizedWeight(torch.from_numpy(w.codes).to(dev), torch.from_numpy(w.scales).to(dev), k, k, 8, k)
    it = _t(dev, idx, torch.int32)
    results = []
    for keep in (True, False):
        xt = _t(dev, x).requires_grad_(True)
        at = _t(dev, a).requires_grad_(True)
        bt = _t(dev, b).requires_grad_(True)
        st = _t(dev, s, torch.float32).requires_grad_(True)
        out = w8.rms_gate_up_lora_swiglu(xt, gamma, wt, at, bt, st, adapter_indices=it, save_projection=keep)
        out.backward(_t(dev, c))
        torch.cuda.synchronize()
        results.append((out.detach(), xt.grad, at.grad, bt.grad, st.grad))
    for kept, recomputed in zip(*results):
        assert torch.equal(kept, recomputed)
    plain = w8.forward(_t(dev, x), wt, _t(dev, a), _t(dev, b), _t(dev, s, torch.float32), adapter_indices=it,
                       rms_gamma=gamma)
    assert torch.equal(w8.swiglu(plain), results[0][0])
    with pytest.raises(ValueError):
        w8.swiglu(plain[:, :12])
    lib = pkg._native.load()
    st_ = lib.mi355_w8a8_swiglu_v1(plain.data_ptr(), plain.data_ptr() + 16, m, n, None)
    assert pkg._native.STATUS[st_] == "ERR_ALIAS"
