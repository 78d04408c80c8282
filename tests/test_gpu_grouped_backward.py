"""GPU parity of the grouped (per-expert) backward through the C ABI: one native call for all groups
against the CPU oracle's per-expert rule (bf16 cotangents to |a - b| <= 2e-2 + 1e-2 |b|), and bit for
bit against one dense backward call per weight over its rows."""

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


def _case(seed, sizes, k, n, rank, gpw, extra_rows=0):
    rng = np.random.default_rng(seed)
    n_groups = len(sizes)
    n_weights = n_groups // gpw
    m = int(sum(sizes)) + extra_rows
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    dy = o.bf16_round(rng.standard_normal((m, n)).astype(F32))
    codes = rng.integers(-127, 128, (n_weights, k, n)).astype(np.int8)
    scales = (rng.uniform(0.2, 1.0, (n_weights, n)) / (127.0 * np.sqrt(k))).astype(F32)
    a = b = s = None
    if rank:
        a = o.bf16_round(rng.standard_normal((n_groups, k, rank)).astype(F32) * 0.1)
        b = o.bf16_round(rng.standard_normal((n_groups, rank, n)).astype(F32) * 0.1)
        s = rng.uniform(0.5, 2.0, n_groups).astype(F32)
    return x, dy, codes, scales, a, b, s


def _oracle(x, dy, sizes, codes, scales, a, b, s, gpw):
    """Per weight: the dense rule over its rows with the groups that share it as adapters."""
    m, k = x.shape
    n = dy.shape[1]
    n_groups = len(sizes)
    dx = np.zeros((m, k), F32)
    da = np.zeros_like(a) if a is not None else None
    db = np.zeros_like(b) if b is not None else None
    ds = np.zeros(n_groups, F32) if a is not None else None
    row = 0
    for wi in range(n_groups // gpw):
        g0 = wi * gpw
        counts = [int(v) for v in sizes[g0:g0 + gpw]]
        rows = sum(counts)
        if rows == 0:
            continue
        sl = slice(row, row + rows)
        w = o.GroupQuantizedWeight(codes=codes[wi], scales=scales[wi][None, :], original_in_features=k,
                                   padded_in_features=k, bits=8, group_size=k)
        if a is None:
            dx[sl] = o.bf16_round(o._mm64(dy[sl], o.pullback_weight(w, True).T))
        else:
            idx = np.repeat(np.arange(gpw), counts)
            out = o.quantized_lora_linear_multi_bwd(x[sl], w, a[g0:g0 + gpw], b[g0:g0 + gpw], s[g0:g0 + gpw], idx,
                                                    dy[sl], relaxed_weight=True)
            dx[sl], da[g0:g0 + gpw], db[g0:g0 + gpw], ds[g0:g0 + gpw] = out
        row += rows
    return dx, da, db, ds


CASES = [
    # sizes, k, n, rank, groups per weight, rows beyond the groups
    ([5, 0, 300, 17], 256, 512, 8, 1, 0),                   # an empty group, a group over one tile
    ([40, 70, 0, 3, 260, 1], 384, 776, 16, 2, 9),           # two groups per weight, ragged columns, spare rows
    ([33] * 8, 200, 264, 5, 1, 0),                          # K, N off the tile sizes, odd rank
    ([700, 20], 512, 1024, 40, 1, 0),                       # rank over 32, several tiles in a weight
    ([3, 0, 0, 9], 128, 256, 0, 1, 4),                      # no LoRA
    ([(i * 7) % 23 for i in range(130)], 256, 384, 4, 1, 0),  # more groups than a dense call has adapters
    # wide K and few rows per weight: the pull-back's 128-row x 512-k tiles, rows at the tile boundary, a last
    # k tile with three of its sixteen blocks
    ([128, 129, 1, 127, 0, 256], 1096, 264, 16, 1, 0),
    ([60, 70, 100, 29, 0, 0, 5, 130], 1024, 320, 8, 2, 3),  # the same tiles with two groups per weight
]


@pytest.mark.parametrize("sizes,k,n,rank,gpw,extra", CASES)
def test_grouped_backward_matches_oracle_and_per_weight_calls(dev, pkg, sizes, k, n, rank, gpw, extra):
    import torch

    w8 = pkg.w8a8_lora
    x, dy, codes, scales, a, b, s = _case(len(sizes) * 31 + k, sizes, k, n, rank, gpw, extra)
    print(f"[case] grouped backward groups={len(sizes)} rows={x.shape[0]} k={k} n={n} rank={rank} gpw={gpw}", flush=True)
    bf = lambda v: None if v is None else torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(torch.bfloat16)
    gw = w8.prepare_grouped_weight(torch.from_numpy(codes).to(dev), torch.from_numpy(scales).to(dev))
    gs = torch.tensor(sizes, dtype=torch.int32, device=dev)
    st = None if s is None else torch.from_numpy(s).to(dev)
    got = w8.grouped_backward(bf(x), bf(dy), gs, gw, bf(a), bf(b), st, groups_per_weight=gpw)
    torch.cuda.synchronize()
    want = _oracle(x, dy, sizes, codes, scales, a, b, s, gpw)
    rep = wc.compare(_np(got[0]), want[0])
    print(f"[grouped backward parity] dx {rep}", flush=True)
    assert rep["violations"] == 0, rep
    if extra:
        assert not _np(got[0])[-extra:].any()
    if rank:
        for name, g, w_ in (("dA", got[1], want[1]), ("dB", got[2], want[2])):
            rep = wc.compare(_np(g), w_)
            print(f"[grouped backward parity] {name} {rep}", flush=True)
            assert rep["violations"] == 0, (name, rep)
        np.testing.assert_allclose(_np(got[3]), want[3], rtol=1e-2, atol=1e-2)
        empty = [g for g, c in enumerate(sizes) if c == 0]
        assert not _np(got[1])[empty].any() and not _np(got[2])[empty].any() and not _np(got[3])[empty].any()
    else:
        assert got[1] is None and got[2] is None and got[3] is None
    # one dense backward call per weight gives the same bits
    ref = w8.grouped_backward_per_weight(bf(x), bf(dy), gs, gw, bf(a), bf(b), st, groups_per_weight=gpw)
    torch.cuda.synchronize()
    assert torch.equal(got[0], ref[0])
    if rank:
        assert torch.equal(got[1], ref[1]) and torch.equal(got[2], ref[2]) and torch.equal(got[3], ref[3])
    # dx alone
    only = w8.grouped_backward(None, bf(dy), gs, gw, bf(a), bf(b), st, groups_per_weight=gpw, need_lora_grads=False)
    torch.cuda.synchronize()
    assert only[1] is None and torch.equal(only[0], got[0])


def test_grouped_linear_through_autograd(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    sizes, k, n, rank = [50, 0, 130, 7], 256, 512, 8
    x, dy, codes, scales, a, b, s = _case(77, sizes, k, n, rank, 1)
    bf = lambda v: torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(torch.bfloat16)
    gw = w8.prepare_grouped_weight(torch.from_numpy(codes).to(dev), torch.from_numpy(scales).to(dev))
    gs = torch.tensor(sizes, dtype=torch.int32, device=dev)
    xt, at, bt = bf(x).requires_grad_(True), bf(a).requires_grad_(True), bf(b).requires_grad_(True)
    st = torch.from_numpy(s).to(dev).requires_grad_(True)
    out = w8.grouped_lora_linear(xt, gs, gw, at, bt, st)
    assert out.requires_grad
    out.backward(bf(dy))
    torch.cuda.synchronize()
    want = _oracle(x, dy, sizes, codes, scales, a, b, s, 1)
    for name, g, w_ in (("dx", xt.grad, want[0]), ("dA", at.grad, want[1]), ("dB", bt.grad, want[2])):
        rep = wc.compare(_np(g), w_)
        assert rep["violations"] == 0, (name, rep)
    np.testing.assert_allclose(_np(st.grad), want[3], rtol=1e-2, atol=1e-2)


def test_grouped_backward_rejects_bad_arguments(dev, pkg):
    import ctypes
    import torch

    w8, nat = pkg.w8a8_lora, pkg._native
    codes = torch.zeros(2, 64, 128, dtype=torch.int8, device=dev)
    scales = torch.ones(2, 128, device=dev)
    gw = w8.prepare_grouped_weight(codes, scales)
    dy = torch.zeros(10, 128, dtype=torch.bfloat16, device=dev)
    gs = torch.tensor([4, 6], dtype=torch.int32, device=dev)
    with pytest.raises(TypeError):
        w8.grouped_backward(None, dy.float(), gs, gw)
    with pytest.raises(ValueError):
        w8.grouped_backward(None, dy[:, :64], gs, gw)
    with pytest.raises(ValueError):
        w8.grouped_backward(None, dy, gs[:1], gw)
    a = torch.zeros(2, 64, 4, dtype=torch.bfloat16, device=dev)
    b = torch.zeros(2, 4, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        w8.grouped_backward(None, dy, gs, gw, a, b, 1.0)           # cotangents wanted, no x
    lib = nat.load()
    assert lib.mi355_w8a8_grouped_bwd_workspace_bytes(10, 64, 128, 2000, 4, 1) == 0
    assert lib.mi355_w8a8_grouped_bwd_workspace_bytes(10, 64, 128, 3, 4, 2) == 0
    p = nat.GroupedBwdProblem()
    p.struct_size = ctypes.sizeof(nat.GroupedBwdProblem) - 8
    assert nat.STATUS[lib.mi355_w8a8_grouped_bwd_v1(ctypes.byref(p), None)] == "ERR_STRUCT"
    p.struct_size = ctypes.sizeof(nat.GroupedBwdProblem)
    p.m, p.k, p.n, p.n_groups = 10, 64, 128, 2
    assert nat.STATUS[lib.mi355_w8a8_grouped_bwd_v1(ctypes.byref(p), None)] == "ERR_NULL"


def test_grouped_backward_at_the_expert_layer_size(dev, pkg):
    """128 experts, 16384 sorted (token, choice) pairs, hidden 2048 -> 1536 gate/up columns, rank 16:
    the native call against the per-weight calls bit for bit, exact linearity in the cotangent (a
    power of two), zero in -> zero out."""
    import torch

    torch.manual_seed(3)
    w8 = pkg.w8a8_lora
    e, m, k, n, r = 128, 16384, 2048, 1536, 16
    print(f"[case] grouped backward expert layer e={e} m={m} k={k} n={n}", flush=True)
    codes = torch.randint(-127, 128, (e, k, n), dtype=torch.int8, device=dev)
    scales = (torch.rand(e, n, device=dev) * 0.8 + 0.2) / (127.0 * k ** 0.5)
    gw = w8.prepare_grouped_weight(codes, scales)
    del codes
    counts = torch.bincount(torch.randint(0, e, (m,), device=dev), minlength=e).to(torch.int32)
    x = torch.randn(m, k, device=dev).to(torch.bfloat16)
    dy = torch.randn(m, n, device=dev).to(torch.bfloat16)
    a = (torch.randn(e, k, r, device=dev) * 0.05).to(torch.bfloat16)
    b = (torch.randn(e, r, n, device=dev) * 0.05).to(torch.bfloat16)
    s = torch.rand(e, device=dev) + 0.5
    got = [t.clone() for t in w8.grouped_backward(x, dy, counts, gw, a, b, s)]
    ref = w8.grouped_backward_per_weight(x, dy, counts, gw, a, b, s)
    torch.cuda.synchronize()
    for g, w_ in zip(got, ref):
        assert torch.equal(g, w_)
    two = w8.grouped_backward(x, 2.0 * dy, counts, gw, a, b, s)
    for g, t in zip(got, two):
        assert torch.equal(2.0 * g.float(), t.float())
    zero = w8.grouped_backward(x, 0.0 * dy, counts, gw, a, b, s)
    torch.cuda.synchronize()
    assert all(not t.any() for t in zero)
