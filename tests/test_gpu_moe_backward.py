"""GPU parity of the expert MLP's backward (through the C ABI): the combine pull-back against the CPU
oracle (bf16 rows to |a - b| <= 2e-2 + 1e-2 |b|, float32 weight cotangents to 1e-3 of their scale) and
the whole chain through autograd against the oracle's chain with the reference's W8A8 gate
(relative L2 < 1e-2, cosine >= 0.9999)."""

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


def _np(v):
    import torch

    return v.detach().to(torch.float32).cpu().numpy()


@pytest.mark.parametrize("t,k,width", [(1, 1, 8), (37, 4, 264), (512, 8, 2048), (5, 64, 16)])
def test_combine_backward_matches_oracle(dev, pkg, t, k, width):
    import torch

    w8 = pkg.w8a8_lora
    rng = np.random.default_rng(t * 7 + width)
    expert_out = o.bf16_round(rng.standard_normal((t * k, width)).astype(F32))
    unsort = rng.permutation(t * k).astype(np.int32)
    sort = np.argsort(unsort).astype(np.int32)
    w = rng.uniform(0.05, 1.0, (t, k)).astype(F32)
    d_out = o.bf16_round(rng.standard_normal((t, width)).astype(F32))
    print(f"[case] combine backward t={t} k={k} width={width}", flush=True)
    bf = lambda v: torch.from_numpy(v).to(dev).to(torch.bfloat16)
    d_e, d_w = w8.moe_combine_backward(bf(d_out), bf(expert_out), torch.from_numpy(sort).to(dev), torch.from_numpy(w).to(dev))
    torch.cuda.synchronize()
    want_e, want_w = o.moe_combine_bwd(d_out, expert_out, unsort, w)
    rep = wc.compare(_np(d_e), want_e)
    assert rep["violations"] == 0 and rep["bitwise_fraction"] > 0.999, rep
    scale = max(float(np.abs(want_w).max()), 1e-3)
    assert np.abs(_np(d_w) - want_w).max() <= 1e-3 * scale
    only, none = w8.moe_combine_backward(bf(d_out), None, torch.from_numpy(sort).to(dev), torch.from_numpy(w).to(dev),
                                         need_weight_grads=False)
    torch.cuda.synchronize()
    assert none is None and torch.equal(only, d_e)


@pytest.mark.parametrize("t,e,k,norm", [(1, 2, 1, True), (37, 12, 4, True), (300, 128, 8, True), (64, 130, 8, False),
                                        (9, 1000, 64, True)])
def test_route_backward_matches_oracle(dev, pkg, t, e, k, norm):
    import torch

    w8 = pkg.w8a8_lora
    rng = np.random.default_rng(t + e)
    logits = (rng.standard_normal((t, e)) * 2.0).astype(F32)
    dw = rng.standard_normal((t, k)).astype(F32)
    print(f"[case] route backward t={t} e={e} k={k} norm={norm}", flush=True)
    lt = torch.from_numpy(logits).to(dev)
    _, sel = w8.moe_route(lt, k, norm)
    got = _np(w8.moe_route_backward(lt, sel, torch.from_numpy(dw).to(dev), norm))
    want = o.moe_route_bwd(logits, sel.cpu().numpy(), dw, norm)
    scale = max(float(np.abs(want).max()), 1e-6)
    assert np.abs(got - want).max() <= 2e-5 * scale + 1e-9, float(np.abs(got - want).max()) / scale
    assert np.abs(got.sum(-1)).max() <= 1e-5 * scale * e ** 0.5     # softmax is shift invariant
    # through autograd, against torch's own derivative of softmax -> gather -> renormalise
    la = lt.clone().requires_grad_(True)
    wts, sel2 = w8._MoeRouteFunction.apply(la, k, norm)
    assert torch.equal(sel2, sel) and not sel2.requires_grad
    wts.backward(torch.from_numpy(dw).to(dev))
    lb = lt.clone().requires_grad_(True)
    ps = torch.softmax(lb, -1).gather(1, sel.to(torch.int64))
    (ps / ps.sum(-1, keepdim=True) if norm else ps).backward(torch.from_numpy(dw).to(dev))
    torch.cuda.synchronize()
    assert float((la.grad - lb.grad).abs().max()) <= 2e-5 * scale + 1e-9


def _mlp_case(seed, t, e, h, inter, r):
    rng = np.random.default_rng(seed)
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    logits = rng.standard_normal((t, e)).astype(F32)
    gu_codes = rng.integers(-127, 128, (e, h, 2 * inter)).astype(np.int8)
    gu_scales = (rng.uniform(0.2, 1.0, (e, 2 * inter)) / (127.0 * np.sqrt(h))).astype(F32)
    dn_codes = rng.integers(-127, 128, (e, inter, h)).astype(np.int8)
    dn_scales = (rng.uniform(0.2, 1.0, (e, h)) / (127.0 * np.sqrt(inter))).astype(F32)
    mk = lambda *shape: o.bf16_round((rng.standard_normal(shape) * 0.1).astype(F32))
    lora = (mk(e, h, r), mk(e, r, 2 * inter), mk(e, inter, r), mk(e, r, h))
    d_out = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    return hidden, logits, gu_codes, gu_scales, dn_codes, dn_scales, lora, d_out


@pytest.mark.parametrize("t,e,k,h,inter,r", [(24, 4, 2, 64, 32, 4), (300, 16, 4, 256, 128, 8), (64, 130, 8, 128, 64, 16)])
def test_expert_mlp_backward_through_autograd(dev, pkg, t, e, k, h, inter, r):
    import torch

    w8 = pkg.w8a8_lora
    hidden, logits, gu_codes, gu_scales, dn_codes, dn_scales, lora, d_out = _mlp_case(t + e, t, e, h, inter, r)
    print(f"[case] expert mlp backward t={t} e={e} k={k} h={h} inter={inter} r={r}", flush=True)
    s = F32(1.25)
    bf = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(torch.bfloat16)
    guw = w8.prepare_grouped_weight(torch.from_numpy(gu_codes).to(dev), torch.from_numpy(gu_scales).to(dev))
    dnw = w8.prepare_grouped_weight(torch.from_numpy(dn_codes).to(dev), torch.from_numpy(dn_scales).to(dev))
    ht = bf(hidden).requires_grad_(True)
    lt = torch.from_numpy(logits).to(dev).requires_grad_(True)
    lora_t = [bf(v).requires_grad_(True) for v in lora]
    st = torch.tensor(float(s), device=dev, requires_grad=True)
    out = w8.w8a8_moe_expert_mlp(ht, lt, k, guw, dnw, *lora_t, st, enabled=True)
    assert out.requires_grad and tuple(out.shape) == (t, h)
    with torch.no_grad():
        plain = w8.w8a8_moe_expert_mlp(ht, lt, k, guw, dnw, *lora_t, st, enabled=True)
    assert torch.equal(plain, out.detach())          # the training forward gives the same bits
    out.backward(bf(d_out))
    torch.cuda.synchronize()
    gu = [o.GroupQuantizedWeight(gu_codes[i], gu_scales[i:i + 1], h, h, 8, h) for i in range(e)]
    dn = [o.GroupQuantizedWeight(dn_codes[i], dn_scales[i:i + 1], inter, inter, 8, inter) for i in range(e)]
    want = o.moe_expert_mlp_bwd(hidden, logits, k, gu, dn, *lora, s, d_out)
    got = {"d_hidden": ht.grad, "d_gate_up_a": lora_t[0].grad, "d_gate_up_b": lora_t[1].grad,
           "d_down_a": lora_t[2].grad, "d_down_b": lora_t[3].grad, "d_router_logits": lt.grad}
    for name, g in got.items():
        gate = o.numerical_gate(_np(g), want[name])
        print(f"[moe backward parity] {name} {gate}", flush=True)
        assert gate["relative_l2"] < 1e-2 and gate["cosine"] >= 0.9999, (name, gate)
    assert abs(float(st.grad) - float(want["d_scaling"])) <= 1e-2 * abs(float(want["d_scaling"])) + 0.05
    # frozen router and hidden rows: only the LoRA factors get cotangents
    lora_2 = [bf(v).requires_grad_(True) for v in lora]
    out2 = w8.w8a8_moe_expert_mlp(bf(hidden), torch.from_numpy(logits).to(dev), k, guw, dnw, *lora_2, float(s), enabled=True)
    out2.backward(bf(d_out))
    torch.cuda.synchronize()
    for a, b in zip(lora_2, lora_t):
        assert torch.equal(a.grad, b.grad)


def test_combine_backward_rejects_bad_arguments(dev, pkg):
    import torch

    w8, nat = pkg.w8a8_lora, pkg._native
    d_out = torch.zeros(4, 16, dtype=torch.bfloat16, device=dev)
    w = torch.ones(4, 2, device=dev)
    sort = torch.arange(8, dtype=torch.int32, device=dev)
    eo = torch.zeros(8, 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(TypeError):
        w8.moe_combine_backward(d_out.float(), eo, sort, w)
    with pytest.raises(ValueError):
        w8.moe_combine_backward(d_out, eo, sort[:4], w)
    with pytest.raises(ValueError):
        w8.moe_combine_backward(d_out, None, sort, w)
    lib = nat.load()
    d_eo = torch.zeros_like(eo)
    st = lib.mi355_w8a8_moe_combine_bwd_v1(d_out.data_ptr(), None, sort.data_ptr(), w.data_ptr(), d_eo.data_ptr(),
                                           w.data_ptr(), 4, 2, 16, None)
    assert nat.STATUS[st] == "ERR_NULL"              # weight cotangent without expert_out
    st = lib.mi355_w8a8_moe_combine_bwd_v1(d_out.data_ptr(), eo.data_ptr(), sort.data_ptr(), w.data_ptr(), eo.data_ptr(),
                                           None, 4, 2, 16, None)
    assert nat.STATUS[st] == "ERR_ALIAS"
    st = lib.mi355_w8a8_moe_combine_bwd_v1(d_out.data_ptr(), eo.data_ptr(), sort.data_ptr(), w.data_ptr(), d_eo.data_ptr(),
                                           None, 4, 2, 12, None)
    assert nat.STATUS[st] == "ERR_SHAPE"
