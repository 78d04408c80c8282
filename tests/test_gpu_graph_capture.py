"""The native calls under HIP graph capture: a plan's ``run()`` neither allocates nor synchronizes nor
records a memset, so a decode loop or a training step can capture it once and replay it.  Every replay
(with eager work and synchronizations between replays, and new operand values in the same buffers)
must reproduce the eager result bit for bit."""

import numpy as np
import pytest

import w8a8_cases as wc

pytestmark = pytest.mark.gpu


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


def _replays(torch, run, outputs, refresh, n=4):
    """Capture ``run`` once; before every replay ``refresh(i)`` rewrites the operands in place, the
    eager call gives the expected outputs, unrelated eager work runs, then the replay must match."""
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run()                                   # warm-up outside the capture, on the capture's stream kind
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run()
    for i in range(n):
        refresh(i)
        run()
        torch.cuda.synchronize()
        want = [t.clone() for t in outputs()]
        for t in outputs():
            t.fill_(7.0) if t.is_floating_point() else t.fill_(7)      # the replay must rewrite everything
        junk = torch.randn(512, 512, device=want[0].device)
        junk = (junk @ junk).sum()              # the program's own eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for j, (g, w) in enumerate(zip(outputs(), want)):
            assert torch.equal(g, w), (i, j)
        assert bool(torch.isfinite(junk))


FORWARD_CASES = [
    # m, k, n, adapters, rank, rms, swiglu, residual
    (16, 1024, 768, 4, 16, False, False, True),      # two-kernel streaming path
    (64, 4096, 1024, 2, 16, True, False, False),     # 32-row chunks of the streaming path
    (96, 4096, 1024, 2, 16, True, False, False),     # 128 x 128 tiles, adapters on block boundaries
    (300, 512, 1024, 3, 32, True, True, False),      # tiled kernel with a persistent schedule
    (1100, 768, 2304, 8, 16, False, False, False),   # several row tiles, per-XCD tile counters
]


@pytest.mark.parametrize("m,k,n,n_ad,rank,rms,swiglu,residual", FORWARD_CASES)
def test_forward_plan_replays(dev, pkg, m, k, n, n_ad, rank, rms, swiglu, residual):
    import torch

    w8 = pkg.w8a8_lora
    print(f"[case] graph forward m={m} k={k} n={n} adapters={n_ad} rms={rms} swiglu={swiglu}", flush=True)
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=rank, seed=m + n, rms=rms, swiglu=swiglu, residual=residual)
    t = wc.to_torch(case, dev)
    res = t.get("residual")
    if swiglu and res is not None:
        res = res[:, : n // 2].contiguous()
    plan = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                          rms_gamma=t.get("gamma"), residual=res, swiglu=swiglu)
    x, idx = plan.x_flat, plan.adapter_indices
    assert x.data_ptr() == t["x"].data_ptr()
    gen = torch.Generator(device=dev).manual_seed(m)

    def refresh(i):
        x.copy_(torch.randn(x.shape, device=dev, generator=gen).to(torch.bfloat16) * (1.0 + i))
        idx.copy_(torch.randint(0, n_ad, idx.shape, device=dev, generator=gen, dtype=torch.int32))

    _replays(torch, plan.run, lambda: [plan.out], refresh)


def test_backward_plan_replays(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    m, k, n, n_ad, rank = 520, 768, 1280, 3, 16
    print(f"[case] graph backward m={m} k={k} n={n}", flush=True)
    case = wc.make_case(m, k, n, n_adapters=n_ad, rank=rank, seed=9)
    t = wc.to_torch(case, dev)
    dy = torch.randn(m, n, device=dev).to(torch.bfloat16)
    plan = w8.BackwardPlan(t["x"], dy, t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"])
    outs = plan.run()
    gen = torch.Generator(device=dev).manual_seed(3)

    def refresh(i):
        dy.copy_(torch.randn(dy.shape, device=dev, generator=gen).to(torch.bfloat16) * (0.5 + i))

    _replays(torch, plan.run, lambda: list(outs), refresh)


def test_qkv_stage_backward_plan_replays(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    hq, hkv, d, rot, k, m, n_ad, rank = 8, 2, 64, 16, 512, 200, 2, 8
    cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000.0, 1e-6)
    print(f"[case] graph qkv backward m={m} k={k} width={cfg.fused_width}", flush=True)
    case = wc.make_case(m, k, cfg.fused_width, n_adapters=n_ad, rank=rank, seed=21, rms=True)
    t = wc.to_torch(case, dev)
    qw, kw = torch.randn(d, device=dev) * 0.1, torch.randn(d, device=dev) * 0.1
    pos = torch.arange(m, dtype=torch.int32, device=dev)
    cots = [torch.randn(m, hq * d, device=dev).to(torch.bfloat16), torch.randn(m, hkv * d, device=dev).to(torch.bfloat16),
            torch.randn(m, hkv * d, device=dev).to(torch.bfloat16), torch.randn(m, hq * d, device=dev).to(torch.bfloat16)]
    plan = w8.QkvStageBackwardPlan(t["x"], t["gamma"] - 1.0, qw, kw, t["weight"], t["a"], t["b"], t["s"], pos, cfg, *cots,
                                   adapter_indices=t["idx"])          # recomputes the projection inside run()
    outs = plan.run()
    gen = torch.Generator(device=dev).manual_seed(4)

    def refresh(i):
        for c in cots:
            c.copy_(torch.randn(c.shape, device=dev, generator=gen).to(torch.bfloat16))

    _replays(torch, plan.run, lambda: list(outs), refresh, n=3)


def test_grouped_backward_plan_replays(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    e, k, n, r = 6, 256, 384, 8
    sizes = [40, 0, 300, 7, 129, 64]
    m = sum(sizes) + 3
    print(f"[case] graph grouped backward groups={e} m={m} k={k} n={n}", flush=True)
    codes = torch.randint(-127, 128, (e, k, n), dtype=torch.int8, device=dev)
    scales = (torch.rand(e, n, device=dev) * 0.8 + 0.2) / (127.0 * k ** 0.5)
    gw = w8.prepare_grouped_weight(codes, scales)
    x = torch.randn(m, k, device=dev).to(torch.bfloat16)
    dy = torch.randn(m, n, device=dev).to(torch.bfloat16)
    a = (torch.randn(e, k, r, device=dev) * 0.1).to(torch.bfloat16)
    b = (torch.randn(e, r, n, device=dev) * 0.1).to(torch.bfloat16)
    gs = torch.tensor(sizes, dtype=torch.int32, device=dev)
    plan = w8.GroupedBackwardPlan(x, dy, gs, gw, a, b, torch.ones(e, device=dev))
    outs = plan.run()
    gen = torch.Generator(device=dev).manual_seed(8)
    layouts = [[40, 0, 300, 7, 129, 64], [0, 0, 1, 500, 0, 39], [90, 90, 90, 90, 90, 90], [540, 0, 0, 0, 0, 0]]

    def refresh(i):
        dy.copy_(torch.randn(dy.shape, device=dev, generator=gen).to(torch.bfloat16))
        plan.group_sizes.copy_(torch.tensor(layouts[i % len(layouts)], dtype=torch.int32))   # the group sizes too

    _replays(torch, plan.run, lambda: list(outs), refresh)


@pytest.mark.parametrize("swiglu,mapped", [(False, False), (True, True)])
def test_grouped_forward_plan_replays(dev, pkg, swiglu, mapped):
    import torch

    w8, native = pkg.w8a8_lora, pkg._native
    e, k, n, r, rep = 6, 256, 384, 8, 2
    layouts = [[40, 0, 300, 7, 129, 64], [0, 0, 1, 500, 0, 39], [90, 90, 90, 90, 90, 90], [540, 0, 0, 0, 0, 0]]
    m = sum(layouts[0]) + 2
    print(f"[case] graph grouped forward groups={e} m={m} k={k} n={n} swiglu={swiglu} row_map={mapped}", flush=True)
    codes = torch.randint(-127, 128, (e, k, n), dtype=torch.int8, device=dev)
    scales = (torch.rand(e, n, device=dev) * 0.8 + 0.2) / (127.0 * k ** 0.5)
    gw = w8.prepare_grouped_weight(codes, scales)
    x = torch.randn(m // rep if mapped else m, k, device=dev).to(torch.bfloat16)
    a = (torch.randn(e, k, r, device=dev) * 0.1).to(torch.bfloat16)
    b = (torch.randn(e, r, n, device=dev) * 0.1).to(torch.bfloat16)
    gs = torch.tensor(layouts[0], dtype=torch.int32, device=dev)
    rmap = torch.randperm(m, device=dev).to(torch.int32) if mapped else None
    plan = w8.GroupedForwardPlan(x, gs, gw, a, b, torch.ones(e, device=dev), swiglu=swiglu, row_map=rmap,
                                 row_repeat=rep if mapped else 1)
    assert plan.x_flat.data_ptr() == x.data_ptr()
    gen = torch.Generator(device=dev).manual_seed(11)

    def refresh(i):
        x.copy_(torch.randn(x.shape, device=dev, generator=gen).to(torch.bfloat16) * (1.0 + i))
        plan.group_sizes.copy_(torch.tensor(layouts[i % len(layouts)], dtype=torch.int32))
        if mapped:
            plan.row_map.copy_(torch.randperm(m, device=dev, generator=gen).to(torch.int32))

    _replays(torch, plan.run, lambda: [plan.out], refresh)
    # the measurement flags: the GEMM kernel alone over the tables the full call left in the workspace
    rows = sum(layouts[3 % len(layouts)])                # the layout of the last replay
    want = plan.run().clone()
    plan.out.fill_(3.0)
    got = plan.run(native.FLAG_SKIP_PROLOGUE)
    torch.cuda.synchronize()
    assert torch.equal(got[:rows], want[:rows])
    assert bool((got[rows:] == 3.0).all())               # the rows past the groups belong to the prologue
    plan.out.fill_(3.0)
    plan.run(native.FLAG_SKIP_GEMM)
    torch.cuda.synchronize()
    assert bool((plan.out[:rows] == 3.0).all()) and bool((plan.out[rows:] == 0).all())
