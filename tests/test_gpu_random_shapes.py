"""Seeded random geometries through the C ABI against the oracle: row counts on both sides of the
decode / tiled switch, K and N tails, ranks 1..64, 1..9 adapters, every optional stage.  The cases
are fixed by their seeds, so a failure names a reproducible shape."""

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


def _geometry(seed, backward=False):
    rng = np.random.default_rng(10_000 + seed)
    m = int(rng.choice([1, 2, 7, 16, 17, 31, 32, 33, 63, 64, 100, 255, 256, 257, 300, 520]))
    k = 8 * int(rng.integers(1, 130))
    n = int(rng.integers(1, 900))
    if backward:
        n = max(8, n // 8 * 8)
    n_ad = int(rng.choice([0, 1, 1, 2, 3, 5, 9]))
    rank = int(rng.choice([1, 3, 8, 16, 17, 32, 33, 64]))
    return rng, m, k, n, n_ad, rank


@pytest.mark.parametrize("seed", range(28))
def test_forward_random_geometry(dev, seed):
    rng, m, k, n, n_ad, rank = _geometry(seed)
    stage = int(rng.integers(0, 4))            # 0 plain, 1 RMSNorm + SwiGLU, 2 residual, 3 RMSNorm only
    swiglu = stage == 1
    if swiglu:
        n += n & 1
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=rank, seed=500 + seed, rms=stage in (1, 3),
                        swiglu=swiglu, residual=stage == 2, student_t=bool(seed & 1),
                        idx_mode="uniform" if seed % 3 else "arange")
    print(f"[case] forward seed={seed} m={m} k={k} n={n} adapters={n_ad} rank={rank} stage={stage}", flush=True)
    got, aux = wc.gpu_forward(case)
    st = wc.oracle_forward(case, return_stages=True)
    if "normalized" in st:
        # codes follow the GPU's own normalized rows: their last float32 bit is not pinned (see the oracle)
        np.testing.assert_array_equal(o.bf16_bits(aux["normalized"]), o.bf16_bits(st["normalized"]))
    np.testing.assert_array_equal(aux["x_codes"], st["x_codes"])
    np.testing.assert_array_equal(aux["x_scales"].view(np.uint32), st["x_scales"].view(np.uint32))
    np.testing.assert_array_equal(aux["acc"], st["acc"])
    rep = wc.compare(got, st["out"])
    assert rep["violations"] == 0, rep


@pytest.mark.parametrize("seed", range(16))
def test_backward_random_geometry(dev, seed):
    import torch

    from __graft_entry__ import load_package

    rng, m, k, n, n_ad, rank = _geometry(100 + seed, backward=True)
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=rank, seed=900 + seed,
                        idx_mode="uniform" if seed % 3 else "arange")
    dy = o.bf16_round(rng.standard_normal((m, n)).astype(F32))
    print(f"[case] backward seed={seed} m={m} k={k} n={n} adapters={n_ad} rank={rank}", flush=True)
    t = wc.to_torch(case, dev)
    w8 = load_package().w8a8_lora
    out = w8.backward(t["x"], torch.from_numpy(dy).to(dev).to(torch.bfloat16), t["weight"], t.get("a"), t.get("b"),
                      t.get("s"), adapter_indices=t.get("idx"))
    torch.cuda.synchronize()
    got = [None if v is None else v.to(torch.float32).cpu().numpy() for v in out]
    if n_ad:
        want = o.quantized_lora_linear_multi_bwd(case["x"], case["weight"], case["a"], case["b"], case["s"],
                                                 case["idx"], dy, relaxed_weight=True)
        for name, u, v in zip(("dx", "dA", "dB"), got, want):
            rep = wc.compare(u, v)
            assert rep["violations"] == 0, (name, rep)
        np.testing.assert_allclose(got[3], want[3], rtol=2e-3, atol=2e-3)
    else:
        want = o.bf16_round(o._mm64(dy, o.pullback_weight(case["weight"], True).T))
        rep = wc.compare(got[0], want)
        assert rep["violations"] == 0, rep
        assert got[1] is None


@pytest.mark.parametrize("seed", range(12))
def test_grouped_random_geometry(dev, seed):
    """Ragged groups (empty ones included), both grouped tile geometries, with and without the row
    map on the way in: integer stages bit-equal to the oracle, outputs within tolerance."""
    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    w8, nat = pkg.w8a8_lora, pkg._native
    rng = np.random.default_rng(20_000 + seed)
    e = int(rng.choice([1, 2, 5, 9]))
    sizes = [int(v) for v in rng.choice([0, 1, 31, 64, 65, 130, 200], e)]
    if sum(sizes) == 0:
        sizes[0] = 3
    k = 8 * int(rng.integers(4, 80))
    n = 2 * int(rng.integers(4, 400))
    rank = int(rng.choice([0, 4, 16, 33]))
    swiglu = bool(seed & 1)
    extra = int(rng.integers(0, 5))
    m = sum(sizes) + extra
    flag = nat.FLAG_GROUPED_TILE64 if seed % 3 == 0 else (nat.FLAG_GROUPED_TILE128 if seed % 3 == 1 else 0)
    print(f"[case] grouped seed={seed} sizes={sizes} k={k} n={n} rank={rank} swiglu={swiglu} flag={flag}", flush=True)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    codes = rng.integers(-127, 128, (e, k, n), dtype=np.int8)
    scales = rng.uniform(0.001, 0.01, (e, n)).astype(F32)
    a = o.bf16_round((rng.standard_normal((e, k, max(rank, 1))) * 0.02).astype(F32))
    b = o.bf16_round((rng.standard_normal((e, max(rank, 1), n)) * 0.02).astype(F32))
    weights = [o.GroupQuantizedWeight(codes[i], scales[i:i + 1], k, k, 8, k) for i in range(e)]
    st = np.concatenate(([0], np.cumsum(sizes)))
    pre = np.zeros((m, n), F32)
    acc = np.zeros((m, n), np.int32)
    xc, xs = o.quantize_rows(x)
    for i, w in enumerate(weights):
        r0, r1 = int(st[i]), int(st[i + 1])
        if r1 > r0:
            pre[r0:r1] = (o.quantized_lora_linear_f32(x[r0:r1], w, a[i], b[i], F32(1.25)) if rank
                          else o.quantized_frozen_linear_f32(x[r0:r1], w))
            acc[r0:r1] = o.int_matmul(xc[r0:r1], codes[i])
    fused = o.bf16_round(pre)
    want = o.swiglu_from_interleaved(fused) if swiglu else fused
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(dev).to(torch.bfloat16)
    gw = w8.prepare_grouped_weight(torch.from_numpy(codes).to(dev), torch.from_numpy(scales).to(dev))
    lora = (bf(a), bf(b), 1.25) if rank else (None, None, None)
    gs = torch.tensor(sizes, dtype=torch.int32)
    out, aux = w8.grouped_forward(bf(x), gs, gw, *lora, swiglu=swiglu, return_aux=True, flags=flag)
    # the same call reading its rows through a map: a permuted copy of x with every row twice
    perm = rng.permutation(m)
    table = np.empty((m, k), F32)
    table[perm] = x
    row_map = torch.from_numpy((2 * perm + rng.integers(0, 2, m)).astype(np.int32)).to(dev)
    mapped = w8.grouped_forward(bf(table), gs, gw, *lora, swiglu=swiglu, flags=flag, row_map=row_map, row_repeat=2)
    torch.cuda.synchronize()
    used = int(st[-1])
    np.testing.assert_array_equal(aux["x_codes"].cpu().numpy(), xc)
    np.testing.assert_array_equal(aux["acc"].cpu().numpy()[:used], acc[:used])
    got = out.float().cpu().numpy()
    assert not got[used:].any()
    rep = wc.compare(got, want)
    assert rep["violations"] == 0, rep
    assert torch.equal(mapped, out)


@pytest.mark.parametrize("seed", range(12))
def test_grouped_backward_random_geometry(dev, seed):
    """The single grouped backward call on ragged groups (empty ones, several groups per weight, spare
    rows): bit-equal to one dense backward call per weight, dx within tolerance of the oracle."""
    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    w8 = pkg.w8a8_lora
    rng = np.random.default_rng(30_000 + seed)
    gpw = int(rng.choice([1, 1, 2, 3]))
    n_weights = int(rng.choice([1, 2, 5, 9, 70]))
    e = gpw * n_weights
    sizes = [int(v) for v in rng.choice([0, 0, 1, 31, 33, 64, 130, 257, 300] if n_weights < 20 else [0, 1, 7, 40], e)]
    if sum(sizes) == 0:
        sizes[-1] = 5
    k = 8 * int(rng.integers(4, 90))
    n = 8 * int(rng.integers(2, 120))
    rank = int(rng.choice([0, 4, 16, 33, 64]))
    extra = int(rng.integers(0, 4))
    m = sum(sizes) + extra
    print(f"[case] grouped backward seed={seed} weights={n_weights} gpw={gpw} rows={m} k={k} n={n} rank={rank}", flush=True)
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(dev).to(torch.bfloat16)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    dy = o.bf16_round(rng.standard_normal((m, n)).astype(F32))
    codes = rng.integers(-127, 128, (n_weights, k, n), dtype=np.int8)
    scales = (rng.uniform(0.2, 1.0, (n_weights, n)) / (127.0 * np.sqrt(k))).astype(F32)
    gw = w8.prepare_grouped_weight(torch.from_numpy(codes).to(dev), torch.from_numpy(scales).to(dev))
    gs = torch.tensor(sizes, dtype=torch.int32, device=dev)
    lora = (None, None, None)
    if rank:
        lora = (bf(rng.standard_normal((e, k, rank)).astype(F32) * 0.1), bf(rng.standard_normal((e, rank, n)).astype(F32) * 0.1),
                torch.from_numpy(rng.uniform(0.5, 2.0, e).astype(F32)).to(dev))
    got = w8.grouped_backward(bf(x), bf(dy), gs, gw, *lora, groups_per_weight=gpw)
    ref = w8.grouped_backward_per_weight(bf(x), bf(dy), gs, gw, *lora, groups_per_weight=gpw)
    torch.cuda.synchronize()
    for g, r in zip(got, ref):
        assert (g is None and r is None) or torch.equal(g, r)
    # dx of the base term against the oracle: per weight dy @ bf16(codes * scales).T (+ the LoRA term)
    st = np.concatenate(([0], np.cumsum(sizes)))
    want = np.zeros((m, k), F32)
    for wi in range(n_weights):
        r0, r1 = int(st[wi * gpw]), int(st[(wi + 1) * gpw])
        if r1 == r0:
            continue
        w = o.GroupQuantizedWeight(codes[wi], scales[wi:wi + 1], k, k, 8, k)
        base = o._mm64(dy[r0:r1], o.pullback_weight(w, True).T)
        if rank:
            a_np, b_np = (v.float().cpu().numpy() for v in lora[:2])
            s_np = lora[2].cpu().numpy()
            for g in range(wi * gpw, (wi + 1) * gpw):
                q0, q1 = int(st[g]) - r0, int(st[g + 1]) - r0
                r_ = (o._mm64(dy[r0:r1][q0:q1], b_np[g].T) * s_np[g]).astype(F32)
                base[q0:q1] = (base[q0:q1] + o._mm64(r_, a_np[g].T)).astype(F32)
        want[r0:r1] = o.bf16_round(base)
    rep = wc.compare(got[0].float().cpu().numpy(), want)
    assert rep["violations"] == 0, rep


@pytest.mark.parametrize("seed", range(10))
def test_group_scaled_random_geometry(dev, seed):
    """W4 / W8 codes with grouped scales, A4 / A8: codes, scales and the float32 base bit-equal."""
    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    rng = np.random.default_rng(30_000 + seed)
    m = int(rng.choice([1, 16, 31, 33, 64, 100, 257]))
    group = 32 * int(rng.choice([1, 2, 3, 4, 8]))
    k = int(rng.integers(1, 6)) * group - int(rng.choice([0, 0, 8, 20]))
    n = int(rng.integers(1, 300))
    wb, ab = int(rng.choice([4, 8])), int(rng.choice([4, 8]))
    n_ad = int(rng.choice([0, 1, 3]))
    rank = int(rng.choice([2, 8, 24, 64]))
    print(f"[case] group-scaled seed={seed} m={m} k={k} n={n} W{wb}A{ab} group={group} adapters={n_ad} rank={rank}",
          flush=True)
    x = o.bf16_round(rng.standard_t(4, (m, k)).astype(F32))
    w = o.quantize_frozen_weight((rng.standard_normal((k, n)) * 0.05).astype(F32), bits=wb, group_size=group,
                                 scale_dtype="f32")
    base, x_codes, x_scales, _ = o.quantized_frozen_linear_f32(x, w, activation_bits=ab, return_parts=True)
    want = base
    args = [None, None, None]
    idx_t = None
    if n_ad:
        a = o.bf16_round((rng.standard_normal((n_ad, k, rank)) * 0.05).astype(F32))
        b = o.bf16_round((rng.standard_normal((n_ad, rank, n)) * 0.05).astype(F32))
        s = rng.uniform(0.5, 2.0, n_ad).astype(F32)
        idx = rng.integers(0, n_ad, m).astype(np.int32)
        want = (base + o.lora_delta_multi(x, a, b, s, idx)).astype(F32)
        bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(dev).to(torch.bfloat16)
        args = [bf(a), bf(b), torch.from_numpy(s).to(dev)]
        idx_t = torch.from_numpy(idx).to(dev)
    wt = pkg.quantized_lora.GroupQuantizedWeight(torch.from_numpy(w.codes).to(dev), torch.from_numpy(w.scales).to(dev),
                                                 k, w.padded_in_features, wb, group)
    got, aux = pkg.gq_linear.forward(torch.from_numpy(x).to(dev).to(torch.bfloat16), wt, *args, activation_bits=ab,
                                     adapter_indices=idx_t, return_aux=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(aux["x_codes"].cpu().numpy(), x_codes.reshape(m, -1))
    np.testing.assert_array_equal(aux["x_scales"].cpu().numpy().view(np.uint32), x_scales.view(np.uint32))
    if m > 32:
        np.testing.assert_array_equal(aux["base"].cpu().numpy().view(np.uint32), base.view(np.uint32))
    else:   # decode kernel: the groups are summed per wave, then the waves (same terms, other order)
        np.testing.assert_allclose(aux["base"].cpu().numpy(), base, rtol=2e-6, atol=1e-6 * float(np.abs(base).max()))
    rep = wc.compare(got.float().cpu().numpy(), o.bf16_round(want))
    assert rep["violations"] == 0, rep
