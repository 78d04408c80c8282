"""GPU parity of the token routing around the grouped expert GEMMs (through the C ABI): route
(softmax / top-k / renormalise), dispatch (stable sort by expert + row gather) and combine.

Index outputs are compared bit for bit with the CPU oracle; the routing weights to 1e-6 relative
(exp and the order of the float32 sums differ in the last bit), the combine bit for bit given the
same inputs (products and sums in float32 in choice order on both sides).
"""

import numpy as np
import pytest

from oracle import w8a8_oracle as o

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


def _bf(dev, v):
    import torch

    return torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(torch.bfloat16)


@pytest.mark.parametrize("t,e,k,norm", [(1, 2, 1, True), (37, 8, 2, True), (300, 128, 8, True), (64, 60, 4, False),
                                        (5, 1024, 64, True), (129, 64, 64, True)])
def test_route_matches_oracle(dev, pkg, t, e, k, norm):
    import torch

    rng = np.random.default_rng(t * 1000 + e)
    logits = (rng.standard_normal((t, e)) * 2.0).astype(F32)
    print(f"[case] moe route t={t} e={e} k={k}", flush=True)
    w, sel = pkg.w8a8_lora.moe_route(torch.from_numpy(logits).to(dev), k, norm)
    torch.cuda.synchronize()
    w, sel = w.cpu().numpy(), sel.cpu().numpy()
    want_w, want_sel = o.moe_route(logits, k, norm)
    differ = np.nonzero((sel != want_sel).any(axis=1))[0]
    # a different choice is only acceptable between experts whose probabilities agree to rounding
    shifted = logits - logits.max(-1, keepdims=True)
    probs = np.exp(shifted.astype(np.float64))
    probs /= probs.sum(-1, keepdims=True)
    for row in differ:
        for a, b in zip(sel[row], want_sel[row]):
            assert abs(probs[row, a] - probs[row, b]) <= 4e-7 * probs[row, b], (row, a, b)
    assert len(differ) <= max(1, t // 100)
    same = np.setdiff1d(np.arange(t), differ)
    np.testing.assert_allclose(w[same], want_w[same], rtol=2e-6, atol=1e-9)
    assert sel.dtype == np.int32 and (np.sort(sel, axis=1)[:, 1:] != np.sort(sel, axis=1)[:, :-1]).all()


def test_route_ties_pick_the_lower_expert(dev, pkg):
    import torch

    logits = np.zeros((3, 16), dtype=F32)
    logits[1, [5, 9]] = 1.0
    logits[2] = np.arange(16)[::-1]
    w, sel = pkg.w8a8_lora.moe_route(torch.from_numpy(logits).to(dev), 3, True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(sel.cpu().numpy(), [[0, 1, 2], [5, 9, 0], [0, 1, 2]])
    np.testing.assert_allclose(w.cpu().numpy().sum(-1), 1.0, rtol=1e-6)
    assert len(set(w[0].tolist())) == 1        # equal probabilities give equal weights


@pytest.mark.parametrize("t,rep,g,h,with_ad", [(1, 1, 1, 8, False), (50, 2, 8, 64, True), (1000, 8, 128, 256, True),
                                               (4099, 1, 1024, 16, False), (700, 4, 3, 520, True),
                                               (33, 3, 5, 2568, False), (257, 8, 16, 4096, False)])
def test_dispatch_matches_oracle(dev, pkg, t, rep, g, h, with_ad):
    import torch

    rng = np.random.default_rng(t + g)
    tokens = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    idx = rng.integers(0, g, t * rep).astype(np.int32)
    if g > 4:
        idx[idx == 2] = 3            # an empty group
    ad = rng.integers(0, 5, t).astype(np.int32) if with_ad else None
    print(f"[case] moe dispatch t={t} repeat={rep} groups={g} width={h}", flush=True)
    got = pkg.w8a8_lora.moe_dispatch(_bf(dev, tokens), torch.from_numpy(idx).to(dev), g, repeat=rep,
                                     adapter_indices=None if ad is None else torch.from_numpy(ad).to(dev))
    torch.cuda.synchronize()
    st, sizes, sort_i, unsort, sad = [None if v is None else v.cpu() for v in got]
    want_t, want_sizes, want_unsort, want_ad = o.prepare_routing(
        np.repeat(tokens, rep, axis=0), idx, g, adapter_indices=None if ad is None else np.repeat(ad, rep))
    np.testing.assert_array_equal(sizes.numpy(), want_sizes)
    np.testing.assert_array_equal(sort_i.numpy(), np.argsort(idx, kind="stable"))
    np.testing.assert_array_equal(unsort.numpy(), want_unsort)
    np.testing.assert_array_equal(st.to(torch.float32).numpy(), want_t)
    if with_ad:
        np.testing.assert_array_equal(sad.numpy(), want_ad)
    else:
        assert sad is None
    if rep == 1:
        ref = pkg.w8a8_lora.prepare_routing(_bf(dev, tokens), torch.from_numpy(idx).to(dev), g,
                                            None if ad is None else torch.from_numpy(ad).to(dev))
        assert torch.equal(ref[0].cpu(), st) and torch.equal(ref[1].cpu(), sizes) and torch.equal(ref[2].cpu(), unsort)
    # indices only
    only = pkg.w8a8_lora.moe_dispatch(None, torch.from_numpy(idx).to(dev), g, repeat=rep)
    assert only[0] is None and torch.equal(only[3].cpu(), unsort)


@pytest.mark.parametrize("t,k,h", [(1, 1, 8), (33, 2, 264), (500, 8, 2048), (7, 64, 16)])
def test_combine_matches_oracle(dev, pkg, t, k, h):
    import torch

    rng = np.random.default_rng(t * 3 + k)
    expert_out = o.bf16_round(rng.standard_normal((t * k, h)).astype(F32))
    unsort = rng.permutation(t * k).astype(np.int32)
    w = rng.uniform(0.0, 1.0, (t, k)).astype(F32)
    print(f"[case] moe combine t={t} k={k} width={h}", flush=True)
    got = pkg.w8a8_lora.moe_combine(_bf(dev, expert_out), torch.from_numpy(unsort).to(dev),
                                    torch.from_numpy(w).to(dev))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(got.to(torch.float32).cpu().numpy(), o.moe_combine(expert_out, unsort, w))


def test_routing_round_trip_full_size(dev, pkg):
    """Qwen3-30B-A3B geometry (4096 tokens, 128 experts, top 8, hidden 2048): dispatch then combine with
    weights 1/top_k of identical rows returns the rows; sizes add up; sortedness."""
    import torch

    torch.manual_seed(3)
    t, e, k, h = 4096, 128, 8, 2048
    print(f"[case] moe routing full size t={t} e={e} k={k} h={h}", flush=True)
    w8 = pkg.w8a8_lora
    logits = torch.randn(t, e, device=dev) * 2
    hidden = torch.randn(t, h, device=dev).to(torch.bfloat16)
    weights, selected = w8.moe_route(logits, k)
    ref_w, ref_sel = torch.topk(torch.softmax(logits, -1), k)
    assert float((selected.long() != ref_sel).float().mean()) < 1e-3
    torch.testing.assert_close(weights.sum(-1), torch.ones(t, device=dev), rtol=1e-5, atol=1e-6)
    xs, sizes, sort_i, unsort, _ = w8.moe_dispatch(hidden, selected, e, repeat=k)
    assert int(sizes.sum()) == t * k
    flat = selected.reshape(-1)
    assert torch.equal(sizes.long(), torch.bincount(flat.long(), minlength=e))
    sorted_experts = flat[sort_i.long()]
    assert bool((sorted_experts[1:] >= sorted_experts[:-1]).all())
    same_expert = sorted_experts[1:] == sorted_experts[:-1]
    assert bool((sort_i[1:][same_expert] > sort_i[:-1][same_expert]).all())       # stable
    assert torch.equal(unsort.long()[sort_i.long()], torch.arange(t * k, device=dev))
    assert torch.equal(xs, hidden[(sort_i // k).long()])
    # powers of two: eight equal rows times 1/8 add up exactly
    back = w8.moe_combine(xs, unsort, torch.full((t, k), 0.125, device=dev))
    assert torch.equal(back, hidden)


def test_routing_rejects_bad_arguments(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    logits = torch.zeros(4, 8, device=dev)
    with pytest.raises(ValueError):
        w8.moe_route(logits, 9)
    with pytest.raises(ValueError):
        w8.moe_route(logits, 0)
    with pytest.raises(ValueError):
        w8.moe_route(logits, True)
    with pytest.raises(pkg._native.NativeError, match="ERR_UNSUPPORTED"):
        w8.moe_route(torch.zeros(4, 2048, device=dev), 2)     # more experts than a wave holds
    idx = torch.zeros(8, dtype=torch.int32, device=dev)
    tok = torch.zeros(4, 16, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        w8.moe_dispatch(tok, idx, 4, repeat=3)
    with pytest.raises(ValueError):
        w8.moe_dispatch(tok[:, :12], idx, 4, repeat=2)
    with pytest.raises(TypeError):
        w8.moe_dispatch(tok.float(), idx, 4, repeat=2)
    with pytest.raises(ValueError):
        w8.moe_dispatch(tok, idx, 2000, repeat=2)
    with pytest.raises(ValueError):
        w8.moe_combine(tok, idx[:4], torch.zeros(2, 4, device=dev))
    lib = pkg._native.load()
    st = lib.mi355_w8a8_moe_combine_v1(tok.data_ptr(), idx.data_ptr(), logits.data_ptr(), tok.data_ptr(), 2, 2, 16, None)
    assert pkg._native.STATUS[st] == "ERR_ALIAS"
    st = lib.mi355_w8a8_moe_route_v1(logits.data_ptr(), 4, 8, 2, 1, logits.data_ptr(), idx.data_ptr(), None)
    assert pkg._native.STATUS[st] == "ERR_ALIAS"


@pytest.mark.parametrize("swiglu,rank", [(True, 16), (False, 0)])
def test_grouped_call_reads_rows_through_the_sort_order(dev, pkg, swiglu, rank):
    """The grouped projection with a row map gives bit for bit what it gives on the gathered copy
    (codes, scales, integer accumulators, output), so the dispatch can skip the row copies."""
    import torch

    rng = np.random.default_rng(17)
    t, h, n, e, topk = 150, 256, 384, 12, 3
    print(f"[case] grouped row map swiglu={swiglu} rank={rank}", flush=True)
    w8 = pkg.w8a8_lora
    hidden = _bf(dev, o.bf16_round(rng.standard_normal((t, h)).astype(F32)))
    selected = torch.from_numpy(np.stack([rng.permutation(e)[:topk] for _ in range(t)]).astype(np.int32)).to(dev)
    codes = torch.from_numpy(rng.integers(-127, 128, (e, h, n), dtype=np.int8)).to(dev)
    scales = torch.from_numpy(rng.uniform(0.001, 0.01, (e, n)).astype(F32)).to(dev)
    weight = w8.prepare_grouped_weight(codes, scales)
    a = b = s = None
    if rank:
        a = _bf(dev, o.bf16_round((rng.standard_normal((e, h, rank)) * 0.05).astype(F32)))
        b = _bf(dev, o.bf16_round((rng.standard_normal((e, rank, n)) * 0.05).astype(F32)))
        s = 1.5
    xs, sizes, sort_i, unsort, _ = w8.moe_dispatch(hidden, selected, e, repeat=topk)
    want, want_aux = w8.grouped_forward(xs, sizes, weight, a, b, s, swiglu=swiglu, return_aux=True)
    got, got_aux = w8.grouped_forward(hidden, sizes, weight, a, b, s, swiglu=swiglu, return_aux=True,
                                      row_map=sort_i, row_repeat=topk)
    torch.cuda.synchronize()
    assert tuple(got.shape) == tuple(want.shape) == (t * topk, n // 2 if swiglu else n)
    assert torch.equal(got, want)
    for key in ("x_codes", "x_scales", "acc"):
        assert torch.equal(got_aux[key], want_aux[key]), key
    with pytest.raises(ValueError):
        w8.grouped_forward(hidden, sizes, weight, a, b, s, row_map=sort_i, row_repeat=0)
    with pytest.raises(ValueError):
        w8.grouped_forward(hidden[:10], sizes, weight, a, b, s, row_map=sort_i, row_repeat=topk)
    # map values outside the rows of x read the nearest row instead of memory beyond x
    wild = sort_i.clone()
    wild[5], wild[77], wild[200] = 2**30, -7, t * topk + 1
    tame = wild.clone()
    tame[5], tame[77], tame[200] = t * topk - 1, 0, t * topk - 1
    got_wild = w8.grouped_forward(hidden, sizes, weight, a, b, s, swiglu=swiglu, row_map=wild, row_repeat=topk)
    got_tame = w8.grouped_forward(hidden, sizes, weight, a, b, s, swiglu=swiglu, row_map=tame, row_repeat=topk)
    torch.cuda.synchronize()
    assert torch.equal(got_wild, got_tame)
