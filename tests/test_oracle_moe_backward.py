"""Pins for the oracle's pull-back of the expert MLP (the derivative of skyrl/tx/models/qwen3.py:172-210):
automatic differentiation in float64 and the identities a wrong index map or a dropped term breaks."""

import numpy as np
import pytest

from oracle import w8a8_oracle as o

F32 = np.float32


def test_combine_pullback_matches_automatic_differentiation():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(4)
    t, k, width = 7, 3, 16
    expert_out = o.bf16_round(rng.standard_normal((t * k, width)).astype(F32))
    unsort = rng.permutation(t * k)
    w = rng.uniform(0.1, 1.0, (t, k)).astype(F32)
    d_out = o.bf16_round(rng.standard_normal((t, width)).astype(F32))
    et = torch.tensor(expert_out.astype(np.float64), requires_grad=True)
    wt = torch.tensor(w.astype(np.float64), requires_grad=True)
    out = (et[torch.tensor(unsort)].reshape(t, k, width) * wt[..., None]).sum(1)
    out.backward(torch.tensor(d_out.astype(np.float64)))
    d_e, d_w = o.moe_combine_bwd(d_out, expert_out, unsort, w)
    assert o.is_bf16_exact(d_e) and d_w.dtype == F32
    ref = et.grad.numpy()
    assert np.all(np.abs(d_e - ref) <= 2.0 ** -8 * np.abs(ref) + 1e-30)
    np.testing.assert_allclose(d_w, wt.grad.numpy(), rtol=2e-6, atol=1e-6)
    # zero in -> zero out; the forward and the pull-back are adjoint in expert_out
    z_e, z_w = o.moe_combine_bwd(0 * d_out, expert_out, unsort, w)
    assert not z_e.any() and not z_w.any()
    fwd = o.moe_combine(expert_out, unsort, w).astype(np.float64)
    assert abs(np.sum(fwd * d_out) - np.sum(expert_out.astype(np.float64) * d_e)) < 0.05 * np.sqrt(np.sum(fwd ** 2) * np.sum(d_out ** 2))


@pytest.mark.parametrize("norm", [True, False])
def test_route_pullback_matches_automatic_differentiation(norm):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(6)
    logits = rng.standard_normal((9, 12)).astype(F32)
    w, sel = o.moe_route(logits, 4, norm)
    dw = rng.standard_normal(w.shape).astype(F32)
    lt = torch.tensor(logits.astype(np.float64), requires_grad=True)
    ps = torch.softmax(lt, -1).gather(1, torch.tensor(sel.astype(np.int64)))
    wt = ps / ps.sum(-1, keepdim=True) if norm else ps
    np.testing.assert_allclose(wt.detach().numpy(), w, rtol=1e-5)
    wt.backward(torch.tensor(dw.astype(np.float64)))
    got = o.moe_route_bwd(logits, sel, dw, norm)
    np.testing.assert_allclose(got, lt.grad.numpy(), rtol=1e-5, atol=1e-7)
    # softmax is shift invariant: the cotangent of every row sums to zero
    assert np.abs(got.sum(-1)).max() < 1e-6
    if norm:  # renormalised weights sum to one: a constant cotangent gives nothing
        assert np.abs(o.moe_route_bwd(logits, sel, np.ones_like(dw), True)).max() < 1e-6


def _case(seed, t=12, e=4, k=2, h=32, inter=16, r=4):
    rng = np.random.default_rng(seed)
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    logits = rng.standard_normal((t, e)).astype(F32)
    gu = [o.quantize_frozen_weight((rng.standard_normal((h, 2 * inter)) * 0.3).astype(F32), bits=8, group_size=h,
                                   scale_dtype="f32") for _ in range(e)]
    dn = [o.quantize_frozen_weight((rng.standard_normal((inter, h)) * 0.3).astype(F32), bits=8, group_size=inter,
                                   scale_dtype="f32") for _ in range(e)]
    mk = lambda *shape: o.bf16_round((rng.standard_normal(shape) * 0.2).astype(F32))
    gua, gub, dna, dnb = mk(e, h, r), mk(e, r, 2 * inter), mk(e, inter, r), mk(e, r, h)
    d_out = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    return hidden, logits, k, gu, dn, gua, gub, dna, dnb, F32(1.5), d_out


@pytest.mark.parametrize("seed", [1, 2])
def test_expert_mlp_backward_matches_automatic_differentiation(seed):
    """The whole rule against autograd through the smooth function (dequantized weights, the selection
    held fixed); the activation quantizers and the bf16 casts between the stages bound the agreement."""
    torch = pytest.importorskip("torch")
    hidden, logits, k, gu, dn, gua, gub, dna, dnb, s, d_out = _case(seed)
    got = o.moe_expert_mlp_bwd(hidden, logits, k, gu, dn, gua, gub, dna, dnb, s, d_out, relaxed_weight=False)
    sel = got["stages"]["selected"]
    t, e = logits.shape
    f64 = lambda v: torch.tensor(np.asarray(v, dtype=np.float64), requires_grad=True)
    ht, lt, guat, gubt, dnat, dnbt, st = f64(hidden), f64(logits), f64(gua), f64(gub), f64(dna), f64(dnb), f64(s)
    wg = torch.tensor(np.stack([o.dequantize_frozen_weight(w) for w in gu]).astype(np.float64))
    wd = torch.tensor(np.stack([o.dequantize_frozen_weight(w) for w in dn]).astype(np.float64))
    ps = torch.softmax(lt, -1).gather(1, torch.tensor(sel.astype(np.int64)))
    wts = ps / ps.sum(-1, keepdim=True)
    out = torch.zeros_like(ht)
    for j in range(k):
        ex = torch.tensor(sel[:, j].astype(np.int64))
        fused = torch.einsum("tk,tkn->tn", ht, wg[ex]) \
            + torch.einsum("tr,trn->tn", torch.einsum("tk,tkr->tr", ht, guat[ex]), gubt[ex]) * st
        act = torch.nn.functional.silu(fused[:, 0::2]) * fused[:, 1::2]
        down = torch.einsum("ti,tin->tn", act, wd[ex]) \
            + torch.einsum("tr,trn->tn", torch.einsum("ti,tir->tr", act, dnat[ex]), dnbt[ex]) * st
        out = out + down * wts[:, j:j + 1]
    out.backward(torch.tensor(d_out.astype(np.float64)))
    refs = {"d_hidden": ht.grad, "d_router_logits": lt.grad, "d_gate_up_a": guat.grad, "d_gate_up_b": gubt.grad,
            "d_down_a": dnat.grad, "d_down_b": dnbt.grad, "d_scaling": st.grad}
    for name, ref in refs.items():
        ref = ref.numpy()
        if name == "d_scaling":  # one scalar: a sum of per-expert terms of size ~10 that partly cancel
            assert abs(float(got[name]) - float(ref)) < 0.05 * abs(float(ref)) + 0.3, (name, got[name], ref)
            continue
        err = np.linalg.norm(np.asarray(got[name], dtype=np.float64) - ref) / np.linalg.norm(ref)
        assert err < 0.05, (name, err)


def test_expert_mlp_backward_chains_and_vanishes():
    hidden, logits, k, gu, dn, gua, gub, dna, dnb, s, d_out = _case(5)
    got = o.moe_expert_mlp_bwd(hidden, logits, k, gu, dn, gua, gub, dna, dnb, s, d_out)
    st = got["stages"]
    d_down, d_w = o.moe_combine_bwd(d_out, st["down"], st["unsort"], st["weights"])
    np.testing.assert_array_equal(d_down, got["d_down"])
    np.testing.assert_array_equal(o.swiglu_pullback_interleaved(st["fused"], got["d_act"]), got["d_fused"])
    zero = o.moe_expert_mlp_bwd(hidden, logits, k, gu, dn, gua, gub, dna, dnb, s, 0 * d_out)
    for name in ("d_hidden", "d_router_logits", "d_gate_up_a", "d_gate_up_b", "d_down_a", "d_down_b"):
        assert not np.asarray(zero[name]).any(), name
    # experts no token chose get no cotangent
    counts = st["group_sizes"]
    for e_ in np.nonzero(counts == 0)[0]:
        assert not got["d_gate_up_a"][e_].any() and not got["d_down_b"][e_].any()
