"""GPU parity of the pull-back of the Qwen3.5 attention input stage (through the C ABI).

The two memory-bound pull-backs (split / Q-K norm / partial RoPE, decoder RMSNorm in the
``1 + weight`` form) are compared with the CPU oracle on the same inputs to
|a - b| <= 2e-2 + 1e-2 |b| for bf16 outputs (float32 arithmetic in the reference's order; sin, cos,
pow and the row sums differ in their last bits), pass-through chunks bitwise, float32 weight
cotangents to 1e-3 of their scale (5e-3 for the head norms, whose terms carry a bf16 rounding).
The whole rule is checked stage by stage on the device's own intermediates and end to end against
the oracle with the reference's W8A8 gate (relative L2 < 1e-2, cosine >= 0.9999).
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


def _weight_close(got, want, what, rel=1e-3):
    scale = max(float(np.abs(want).max()), 1e-3)
    assert np.abs(got - want).max() <= rel * scale + 1e-5, (what, float(np.abs(got - want).max()), scale)


# The head-norm weight cotangents sum bf16-rounded unrotated cotangents: at large positions one ulp of
# the float32 angle (pow, division) moves sin and cos by 1e-3 and with them many of those roundings.
HEAD = 5e-3


@pytest.mark.parametrize("hq,hkv,d,rot,rows", [(4, 2, 4, 2, 6), (16, 4, 256, 64, 40), (8, 8, 128, 128, 33),
                                               (6, 2, 64, 0, 17), (2, 1, 130, 26, 9), (32, 8, 128, 64, 1500),
                                               (2, 2, 512, 512, 5)])
def test_split_norm_rope_backward_matches_oracle(dev, pkg, hq, hkv, d, rot, rows):
    import torch

    w8 = pkg.w8a8_lora
    cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000.0, 1e-6)
    kw_cfg = dict(num_query_heads=hq, num_kv_heads=hkv, head_dim=d, rotary_dim=rot, rope_theta=10_000.0, eps=1e-6)
    rng = np.random.default_rng(hq * 1000 + d + rows)
    fused = o.bf16_round(rng.standard_normal((rows, cfg.fused_width)).astype(F32) * 2.0)
    qw, kw = (rng.standard_normal(d).astype(F32) * 0.1 for _ in range(2))
    pos = rng.integers(0, 40_000, rows).astype(np.int32)
    pos[0] = 0
    dq = o.bf16_round(rng.standard_normal((rows, hq, d)).astype(F32))
    dk = o.bf16_round(rng.standard_normal((rows, hkv, d)).astype(F32))
    dv = o.bf16_round(rng.standard_normal((rows, hkv, d)).astype(F32))
    dgate = o.bf16_round(rng.standard_normal((rows, hq * d)).astype(F32))
    print(f"[case] qkv post backward hq={hq} hkv={hkv} d={d} rot={rot} rows={rows}", flush=True)
    want, want_qw, want_kw = o.qkv_split_norm_rope_bwd(fused, qw, kw, pos, dq, dk, dv, dgate, **kw_cfg)
    args = (_t(dev, fused), _t(dev, qw, torch.float32), _t(dev, kw, torch.float32), _t(dev, pos, torch.int32), cfg,
            _t(dev, dq), _t(dev, dk), _t(dev, dv), _t(dev, dgate))
    got, none_q, none_k = w8.qkv_split_norm_rope_backward(*args)
    torch.cuda.synchronize()
    assert none_q is None and none_k is None and tuple(got.shape) == fused.shape
    got = _np(got)
    rep = wc.compare(got, want)
    print(f"[qkv backward parity] dfused {rep}", flush=True)
    assert rep["violations"] == 0, rep
    # gate and v cotangents are copied to their chunks bit for bit
    _, _, v_chunks = o.split(got, (hq // hkv * 2 * d, d, d))
    np.testing.assert_array_equal(v_chunks.reshape(rows, hkv, d), dv)
    q_chunks, _, _ = o.split(got, (hq // hkv * 2 * d, d, d))
    np.testing.assert_array_equal(q_chunks.reshape(rows, hq, 2 * d)[..., d:].reshape(rows, hq * d), dgate)
    # with the weight cotangents: the same d_fused, sums over rows and heads in float32
    got2, got_qw, got_kw = w8.qkv_split_norm_rope_backward(*args, need_norm_weight_grads=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(_np(got2), got)
    _weight_close(_np(got_qw), want_qw, "d_q_norm_weight", HEAD)
    _weight_close(_np(got_kw), want_kw, "d_k_norm_weight", HEAD)
    # a missing cotangent counts as zero
    got3, _, _ = w8.qkv_split_norm_rope_backward(*args[:5], None, args[6], None, args[8])
    want3, _, _ = o.qkv_split_norm_rope_bwd(fused, qw, kw, pos, 0 * dq, dk, 0 * dv, dgate, **kw_cfg)
    rep = wc.compare(_np(got3), want3)
    assert rep["violations"] == 0, rep


@pytest.mark.parametrize("m,k,eps", [(1, 8, 1e-6), (19, 1000, 1e-6), (300, 2560, 1e-6), (7, 37, 1e-5), (3, 12288, 1e-6)])
def test_delta_rms_norm_backward_matches_oracle(dev, pkg, m, k, eps):
    import torch

    rng = np.random.default_rng(m * 7 + k)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32) * 2.0)
    w = (0.2 * rng.standard_normal(k)).astype(F32)
    dn = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    print(f"[case] delta rms norm backward m={m} k={k}", flush=True)
    want, want_w = o.delta_rms_norm_vjp(x, w, dn, eps)
    xt, gt, dt = _t(dev, x), _t(dev, (F32(1.0) + w).astype(F32), torch.float32), _t(dev, dn)
    got, got_w = pkg.w8a8_lora.delta_rms_norm_backward(xt, gt, dt, eps=eps, need_weight_grad=True)
    torch.cuda.synchronize()
    rep = wc.compare(_np(got), want)
    print(f"[qkv backward parity] delta rms m{m}k{k} {rep}", flush=True)
    assert rep["violations"] == 0, rep
    assert rep["bitwise_fraction"] > 0.98, rep
    _weight_close(_np(got_w), want_w, "d_weight")
    assert torch.equal(dt, _t(dev, dn))
    same, none_w = pkg.w8a8_lora.delta_rms_norm_backward(xt, gt, dt, eps=eps, in_place=True)
    torch.cuda.synchronize()
    assert none_w is None and same.data_ptr() == dt.data_ptr() and torch.equal(same, got)


def _stage_case(seed, hq, hkv, d, k, batch, seq, rank, n_ad):
    rng = np.random.default_rng(seed)
    width = hq * 2 * d + 2 * hkv * d
    hidden = o.bf16_round(rng.standard_normal((batch, seq, k)).astype(F32))
    inw, qw, kw = (rng.standard_normal(n).astype(F32) * 0.1 for n in (k, d, d))
    wq = o.quantize_frozen_weight(rng.standard_normal((k, width)).astype(F32) * 0.2, bits=8, group_size=k,
                                  scale_dtype="f32")
    a = o.bf16_round(rng.standard_normal((n_ad, k, rank)).astype(F32) * 0.1)
    b = o.bf16_round(rng.standard_normal((n_ad, rank, width)).astype(F32) * 0.1)
    s = rng.uniform(0.5, 1.5, n_ad).astype(F32)
    idx = rng.integers(0, n_ad, batch).astype(np.int32)
    pos = (np.arange(seq)[None, :] + 7 * np.arange(batch)[:, None]).astype(np.int32)
    m = batch * seq
    cots = (o.bf16_round(rng.standard_normal((m, hq, d)).astype(F32)),
            o.bf16_round(rng.standard_normal((m, hkv, d)).astype(F32)),
            o.bf16_round(rng.standard_normal((m, hkv, d)).astype(F32)),
            o.bf16_round(rng.standard_normal((m, hq * d)).astype(F32)))
    return hidden, inw, qw, kw, wq, a, b, s, idx, pos, cots


STAGE_CASES = [
    # hq, hkv, d, rot, k, batch, seq, rank, adapters
    (4, 2, 8, 4, 64, 2, 5, 3, 2),
    (8, 2, 128, 32, 512, 2, 24, 16, 2),
    (16, 4, 256, 64, 1024, 3, 50, 8, 3),
]


@pytest.mark.parametrize("save_projection", [True, False])
@pytest.mark.parametrize("hq,hkv,d,rot,k,batch,seq,rank,n_ad", STAGE_CASES)
def test_stage_backward_through_autograd(dev, pkg, hq, hkv, d, rot, k, batch, seq, rank, n_ad, save_projection):
    import torch

    w8, ql = pkg.w8a8_lora, pkg.quantized_lora
    cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000.0, 1e-6)
    kw_cfg = dict(num_query_heads=hq, num_kv_heads=hkv, head_dim=d, rotary_dim=rot, rope_theta=10_000.0, eps=1e-6)
    hidden, inw, qw, kw, wq, a, b, s, idx, pos, cots = _stage_case(hq + d + k, hq, hkv, d, k, batch, seq, rank, n_ad)
    m = batch * seq
    print(f"[case] qkv stage backward hq={hq} d={d} k={k} m={m} saved={save_projection}", flush=True)
    wt = ql.GroupQuantizedWeight(torch.from_numpy(wq.codes).to(dev), torch.from_numpy(wq.scales).to(dev), k, k, 8, k)
    ht = _t(dev, hidden).requires_grad_(True)
    inwt, qwt, kwt = (_t(dev, v, torch.float32).requires_grad_(True) for v in (inw, qw, kw))
    at, bt = _t(dev, a).requires_grad_(True), _t(dev, b).requires_grad_(True)
    st = _t(dev, s, torch.float32).requires_grad_(True)
    it, pt = _t(dev, idx, torch.int32), _t(dev, pos, torch.int32)
    outs = w8.w8a8_qkv_lora_rope(ht, inwt, qwt, kwt, wt, at, bt, st, pt, config=cfg, adapter_indices=it,
                                 enabled=True, save_projection=save_projection)
    rows_idx = np.repeat(idx, seq)
    want_fwd = o.w8a8_qkv_lora_rope(hidden.reshape(m, k), inw, qw, kw, wq, a, b, s, rows_idx, pos.reshape(-1), **kw_cfg)
    for u, w_ in zip(outs, want_fwd):
        assert u.requires_grad
        rep = wc.compare(_np(u).reshape(w_.shape), w_)
        assert rep["violations"] == 0, rep
    shapes = ((batch, seq, hq, d), (batch, seq, hkv, d), (batch, seq, hkv, d), (batch, seq, hq * d))
    torch.autograd.backward(list(outs), [_t(dev, c).reshape(sh) for c, sh in zip(cots, shapes)])
    torch.cuda.synchronize()
    want = o.w8a8_qkv_lora_rope_bwd(hidden.reshape(m, k), inw, qw, kw, wq, a, b, s, rows_idx, pos.reshape(-1), *cots,
                                    relaxed_weight=True, **kw_cfg)
    got = {"dhidden": _np(ht.grad).reshape(m, k), "d_lora_a": _np(at.grad), "d_lora_b": _np(bt.grad)}
    for name, g in got.items():
        gate = o.numerical_gate(g, want[name])
        print(f"[qkv backward parity] m{m}k{k} {name} {gate}", flush=True)
        assert gate["relative_l2"] < 1e-2 and gate["cosine"] >= 0.9999, (name, gate)
    np.testing.assert_allclose(_np(st.grad), want["d_lora_scaling"], rtol=1e-2, atol=1e-2)
    for name, g in (("d_input_norm_weight", inwt.grad), ("d_q_norm_weight", qwt.grad), ("d_k_norm_weight", kwt.grad)):
        gate = o.numerical_gate(_np(g), want[name])
        assert gate["relative_l2"] < 1e-2 and gate["cosine"] >= 0.9999, (name, gate)

    # stage by stage on the device's own intermediates
    gamma = (F32(1.0) + inw).astype(F32)
    fused_dev, aux = w8.forward(_t(dev, hidden.reshape(m, k)), wt, _t(dev, a), _t(dev, b), _t(dev, s, torch.float32),
                                adapter_indices=_t(dev, rows_idx, torch.int32), rms_gamma=_t(dev, gamma, torch.float32),
                                eps=1e-6, return_aux=True)
    fused_np, norm_np = _np(fused_dev), _np(aux["normalized"])
    d_fused_dev, dqw_dev, dkw_dev = w8.qkv_split_norm_rope_backward(
        fused_dev, _t(dev, qw, torch.float32), _t(dev, kw, torch.float32), pt.reshape(-1), cfg,
        *(_t(dev, c) for c in cots), need_norm_weight_grads=True)
    ref_df, ref_qw, ref_kw = o.qkv_split_norm_rope_bwd(fused_np, qw, kw, pos.reshape(-1), *cots, **kw_cfg)
    rep = wc.compare(_np(d_fused_dev), ref_df)
    assert rep["violations"] == 0, rep
    _weight_close(_np(dqw_dev), ref_qw, "d_q_norm_weight", HEAD)
    _weight_close(_np(dkw_dev), ref_kw, "d_k_norm_weight", HEAD)
    np.testing.assert_array_equal(_np(dqw_dev), _np(qwt.grad))        # the rule is exactly this chain
    dn_dev, da_dev, db_dev, _ = w8.backward(aux["normalized"], d_fused_dev, wt, _t(dev, a), _t(dev, b),
                                            _t(dev, s, torch.float32), adapter_indices=_t(dev, rows_idx, torch.int32))
    ref_mid = o.quantized_lora_linear_multi_bwd(norm_np, wq, a, b, s, rows_idx, _np(d_fused_dev), relaxed_weight=True)
    for g, ref, name in zip((dn_dev, da_dev, db_dev), ref_mid[:3], ("dn", "dA", "dB")):
        rep = wc.compare(_np(g), ref)
        assert rep["violations"] == 0, (name, rep)
    np.testing.assert_array_equal(_np(da_dev), got["d_lora_a"])
    dh_dev, dinw_dev = w8.delta_rms_norm_backward(_t(dev, hidden.reshape(m, k)), _t(dev, gamma, torch.float32), dn_dev,
                                                  eps=1e-6, need_weight_grad=True)
    ref_dh, ref_dinw = o.delta_rms_norm_vjp(hidden.reshape(m, k), inw, _np(dn_dev), 1e-6)
    rep = wc.compare(_np(dh_dev), ref_dh)
    assert rep["violations"] == 0, rep
    _weight_close(_np(dinw_dev), ref_dinw, "d_input_norm_weight")
    np.testing.assert_array_equal(_np(dh_dev), got["dhidden"])
    np.testing.assert_array_equal(_np(dinw_dev), _np(inwt.grad))


def test_stage_frozen_norms_and_no_adapters(dev, pkg):
    """LoRA training leaves the norm weights frozen: no weight cotangents are formed; without
    adapters only the hidden rows get one; without gradients the forward alone runs."""
    import torch

    w8, ql = pkg.w8a8_lora, pkg.quantized_lora
    hq, hkv, d, rot, k, batch, seq, rank, n_ad = 8, 2, 64, 16, 256, 2, 9, 4, 2
    cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000.0, 1e-6)
    kw_cfg = dict(num_query_heads=hq, num_kv_heads=hkv, head_dim=d, rotary_dim=rot, rope_theta=10_000.0, eps=1e-6)
    hidden, inw, qw, kw, wq, a, b, s, idx, pos, cots = _stage_case(5, hq, hkv, d, k, batch, seq, rank, n_ad)
    m = batch * seq
    wt = ql.GroupQuantizedWeight(torch.from_numpy(wq.codes).to(dev), torch.from_numpy(wq.scales).to(dev), k, k, 8, k)
    inwt, qwt, kwt = (_t(dev, v, torch.float32) for v in (inw, qw, kw))
    pt = _t(dev, pos, torch.int32)
    at, bt = _t(dev, a).requires_grad_(True), _t(dev, b).requires_grad_(True)
    ht = _t(dev, hidden)
    q, kk, v, gate = w8.w8a8_qkv_lora_rope(ht, inwt, qwt, kwt, wt, at, bt, _t(dev, s, torch.float32), pt, config=cfg,
                                           adapter_indices=_t(dev, idx, torch.int32), enabled=True)
    # only q and gate feed the loss: the k and v cotangents are absent
    torch.autograd.backward([q, gate], [_t(dev, cots[0]).reshape(q.shape), _t(dev, cots[3]).reshape(gate.shape)])
    torch.cuda.synchronize()
    assert ht.grad is None and inwt.grad is None and qwt.grad is None
    want = o.w8a8_qkv_lora_rope_bwd(hidden.reshape(m, k), inw, qw, kw, wq, a, b, s, np.repeat(idx, seq), pos.reshape(-1),
                                    cots[0], 0 * cots[1], 0 * cots[2], cots[3], **kw_cfg)
    for name, g in (("d_lora_a", at.grad), ("d_lora_b", bt.grad)):
        gate_ = o.numerical_gate(_np(g), want[name])
        assert gate_["relative_l2"] < 1e-2 and gate_["cosine"] >= 0.9999, (name, gate_)
    # no adapters
    h2 = _t(dev, hidden).requires_grad_(True)
    outs = w8.w8a8_qkv_lora_rope(h2, inwt, qwt, kwt, wt, None, None, None, pt, config=cfg, enabled=True)
    torch.autograd.backward(list(outs), [_t(dev, c).reshape(u.shape) for c, u in zip(cots, outs)])
    torch.cuda.synchronize()
    base = o.w8a8_qkv_lora_rope_bwd(hidden.reshape(m, k), inw, qw, kw, wq, None, None, None, None, pos.reshape(-1),
                                    *cots, **kw_cfg)
    gate_ = o.numerical_gate(_np(h2.grad).reshape(m, k), base["dhidden"])
    assert gate_["relative_l2"] < 1e-2 and gate_["cosine"] >= 0.9999, gate_
    with torch.no_grad():
        plain = w8.w8a8_qkv_lora_rope(h2, inwt, qwt, kwt, wt, None, None, None, pt, config=cfg, enabled=True)
    assert not plain[0].requires_grad and torch.equal(plain[0], outs[0].detach())


def test_qkv_backward_rejects_bad_arguments(dev, pkg):
    import ctypes
    import torch

    w8, nat = pkg.w8a8_lora, pkg._native
    cfg = w8.Qwen35QKVStageConfig(4, 2, 8, 4, 1e4, 1e-6)
    fused = torch.zeros(3, cfg.fused_width, dtype=torch.bfloat16, device=dev)
    wgt = torch.zeros(8, device=dev)
    pos = torch.zeros(3, dtype=torch.int32, device=dev)
    dq = torch.zeros(3, 4, 8, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        w8.qkv_split_norm_rope_backward(fused, wgt, wgt, pos, cfg, dq[:2], None, None, None)
    with pytest.raises(TypeError):
        w8.qkv_split_norm_rope_backward(fused, wgt, wgt, pos, cfg, dq.float(), None, None, None)
    with pytest.raises(ValueError):
        w8.qkv_split_norm_rope_backward(fused, wgt, wgt, pos[:2], cfg, dq, None, None, None)
    g = torch.ones(16, dtype=torch.float32, device=dev)
    f = torch.zeros(4, 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        w8.delta_rms_norm_backward(f, g, f.clone(), need_weight_grad=True, in_place=True)
    with pytest.raises(ValueError):
        w8.delta_rms_norm_backward(f, g[:8], f.clone())
    lib = nat.load()
    f2 = f.clone()
    dw = torch.zeros(16, device=dev)
    ws = torch.zeros(int(lib.mi355_w8a8_delta_rms_norm_bwd_workspace_bytes(4, 16)), dtype=torch.uint8, device=dev)
    st = lib.mi355_w8a8_delta_rms_norm_bwd_v1(f.data_ptr(), g.data_ptr(), f2.data_ptr(), f2.data_ptr(), dw.data_ptr(),
                                              ws.data_ptr(), ws.numel(), 4, 16, 1e-6, None)
    assert nat.STATUS[st] == "ERR_ALIAS"            # weight cotangent wanted, d_x over d_normalized
    out = torch.zeros_like(f)
    st = lib.mi355_w8a8_delta_rms_norm_bwd_v1(f.data_ptr(), g.data_ptr(), f2.data_ptr(), out.data_ptr(), dw.data_ptr(),
                                              ws.data_ptr(), ws.numel() - 1, 4, 16, 1e-6, None)
    assert nat.STATUS[st] == "ERR_WORKSPACE"
    p = nat.QkvPostBwdProblem()
    p.struct_size = ctypes.sizeof(nat.QkvPostBwdProblem) - 8
    assert nat.STATUS[lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1(ctypes.byref(p), None)] == "ERR_STRUCT"
    p.struct_size = ctypes.sizeof(nat.QkvPostBwdProblem)
    p.m, p.num_query_heads, p.num_kv_heads, p.head_dim, p.rotary_dim = 3, 4, 2, 8, 4
    p.rope_theta, p.rms_eps = 1e4, 1e-6
    assert nat.STATUS[lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1(ctypes.byref(p), None)] == "ERR_NULL"
    p.head_dim = 1024
    assert nat.STATUS[lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1(ctypes.byref(p), None)] == "ERR_UNSUPPORTED"


def test_qkv_backward_full_size_properties(dev, pkg):
    """Qwen3.5-4B attention input stage at M = 2048 rows: the pull-back against float32 torch
    autograd through the same smooth function on the device, linearity in the cotangent (a power
    of two passes through unchanged), zero in -> zero out."""
    import torch

    torch.manual_seed(11)
    hq, hkv, d, rot, m = 16, 4, 256, 64, 2048
    w8 = pkg.w8a8_lora
    cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000_000.0, 1e-6)
    print(f"[case] qkv backward full size m={m} width={cfg.fused_width}", flush=True)
    fused = (torch.randn(m, cfg.fused_width, device=dev) * 2.0).to(torch.bfloat16)
    qw, kw = torch.randn(d, device=dev) * 0.1, torch.randn(d, device=dev) * 0.1
    pos = torch.arange(m, dtype=torch.int32, device=dev)
    cots = [torch.randn(m, hq, d, device=dev).to(torch.bfloat16), torch.randn(m, hkv, d, device=dev).to(torch.bfloat16),
            torch.randn(m, hkv, d, device=dev).to(torch.bfloat16), torch.randn(m, hq * d, device=dev).to(torch.bfloat16)]
    got, gqw, gkw = w8.qkv_split_norm_rope_backward(fused, qw, kw, pos, cfg, *cots, need_norm_weight_grads=True)

    f32 = fused.float().requires_grad_(True)
    qw32, kw32 = qw.clone().requires_grad_(True), kw.clone().requires_grad_(True)
    grouped = f32.reshape(m, hkv, (hq // hkv * 2 + 2) * d)
    qg = grouped[..., :hq // hkv * 2 * d].reshape(m, hq, 2 * d)

    def norm(x, w):
        return x * torch.rsqrt((x * x).mean(-1, keepdim=True) + 1e-6) * (1.0 + w)

    def rope(x):
        half = rot // 2
        frac = 2.0 * torch.arange(half, dtype=torch.float32, device=dev) / rot
        ang = pos.float()[:, None] / torch.pow(torch.tensor(10_000_000.0, device=dev), frac)
        sin, cos = torch.sin(ang)[:, None, :], torch.cos(ang)[:, None, :]
        first, second = x[..., :half], x[..., half:rot]
        return torch.cat([first * cos - second * sin, first * sin + second * cos, x[..., rot:]], dim=-1)

    q = rope(norm(qg[..., :d], qw32))
    gate = qg[..., d:].reshape(m, hq * d)
    kk = rope(norm(grouped[..., hq // hkv * 2 * d:hq // hkv * 2 * d + d], kw32))
    v = grouped[..., hq // hkv * 2 * d + d:]
    torch.autograd.backward([q, kk, v, gate], [c.float() for c in cots])
    ref = f32.grad
    bad = (got.float() - ref).abs() > 2e-2 + 1e-2 * ref.abs()
    assert int(bad.sum()) == 0, int(bad.sum())
    for g, r in ((gqw, qw32.grad), (gkw, kw32.grad)):
        assert float((g - r).abs().max()) <= 2e-2 * float(r.abs().max())     # bf16 rounding of the unrotated dy
    two, _, _ = w8.qkv_split_norm_rope_backward(fused, qw, kw, pos, cfg, *(2.0 * c for c in cots))
    assert torch.equal(two.float(), 2.0 * got.float())
    zero, zq, zk = w8.qkv_split_norm_rope_backward(fused, qw, kw, pos, cfg, *(0.0 * c for c in cots),
                                                   need_norm_weight_grads=True)
    torch.cuda.synchronize()
    assert not zero.any() and not zq.any() and not zk.any()
