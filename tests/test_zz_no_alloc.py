"""mi355_w8a8_forward_static_ws_v1: the forward call on the library's own static workspace.

Called through the C ABI and held to the existing entry point's results (bit for bit: same kernels,
another workspace) and to the oracle's tolerance, on two calls in a row, the second with a smaller
input, so that whatever the first call left in the shared array is shown not to leak into the second.
"""

import ctypes

import numpy as np
import pytest

import w8a8_cases as wc

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def pkg():
    from __graft_entry__ import load_package

    return load_package()


def _static_ws_forward(pkg, plan):
    """Run plan's problem through the static-workspace entry point into a fresh output tensor."""
    import torch

    native = pkg._native
    lib = native.load()
    p = native.Problem()
    ctypes.memmove(ctypes.byref(p), ctypes.byref(plan.problem), ctypes.sizeof(p))
    out = torch.full_like(plan.out, float("nan"))
    p.out = out.data_ptr()
    p.workspace = None
    p.workspace_bytes = 0
    p.aux_x_codes = p.aux_x_scales = p.aux_acc = p.aux_normalized = None
    with torch.cuda.device(plan.device):
        status = lib.mi355_w8a8_forward_static_ws_v1(ctypes.byref(p), int(torch.cuda.current_stream().cuda_stream))
    native.check("mi355_w8a8_forward_static_ws_v1", status)
    return out


@pytest.mark.parametrize("shapes", [
    # (first call, second and smaller call)
    (dict(m=700, k=1024, n=1536, n_adapters=4, rank=32, rms=True, swiglu=True),
     dict(m=130, k=512, n=768, n_adapters=2, rank=16, rms=True, swiglu=True)),
    (dict(m=16, k=2048, n=1024, n_adapters=8, rank=32, residual=True, idx_mode="arange"),
     dict(m=5, k=512, n=256, n_adapters=3, rank=8, residual=True, idx_mode="arange")),
    (dict(m=300, k=640, n=520, n_adapters=0), dict(m=40, k=256, n=260, n_adapters=0)),
])
def test_static_workspace_matches_caller_workspace(pkg, shapes):
    import torch

    dev = torch.device("cuda:0")
    w8 = pkg.w8a8_lora
    for i, shape in enumerate(shapes):
        shape = dict(shape)
        m, k, n = shape.pop("m"), shape.pop("k"), shape.pop("n")
        print(f"[case] static workspace call {i}: {m}x{k}x{n} {shape}", flush=True)
        case = wc.make_case(m, k, n, seed=41 + i, **shape)
        t = wc.to_torch(case, dev)
        plan = w8.ForwardPlan(t["x"], t["weight"], t.get("a"), t.get("b"), t.get("s"),
                              adapter_indices=t.get("idx"), rms_gamma=t.get("gamma"), eps=1e-6,
                              residual=t.get("residual"), swiglu=bool(case.get("swiglu")))
        want_gpu = plan.run().clone()
        got = _static_ws_forward(pkg, plan)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want_gpu.view(torch.int16))
        rep = wc.compare(got.to(torch.float32).cpu().numpy().reshape(m, -1), wc.oracle_forward(case))
        assert rep["violations"] == 0, rep


def test_static_workspace_allocates_nothing_and_replays_under_capture(pkg):
    """After the first call on a device (which looks the array's address up) a call leaves the free device
    memory as it found it, and a call captured into a HIP graph replays with the eager call's bits."""
    import torch

    dev = torch.device("cuda:0")
    w8 = pkg.w8a8_lora
    case = wc.make_case(260, 512, 520, n_adapters=3, rank=16, seed=47, residual=True)
    t = wc.to_torch(case, dev)
    plan = w8.ForwardPlan(t["x"], t["weight"], t["a"], t["b"], t["s"], adapter_indices=t["idx"],
                          residual=t["residual"])
    want = plan.run().clone()
    first = _static_ws_forward(pkg, plan)  # warm-up: resolves the symbol's address
    torch.cuda.synchronize()
    native = pkg._native
    lib = native.load()
    p = native.Problem()
    ctypes.memmove(ctypes.byref(p), ctypes.byref(plan.problem), ctypes.sizeof(p))
    out = torch.full_like(plan.out, float("nan"))
    p.out = out.data_ptr()
    p.workspace, p.workspace_bytes = None, 0
    p.aux_x_codes = p.aux_x_scales = p.aux_acc = p.aux_normalized = None
    stream = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(stream):  # (the runtime sets a new stream's own resources up at its first launch)
        assert lib.mi355_w8a8_forward_static_ws_v1(ctypes.byref(p), int(stream.cuda_stream)) == 0
    stream.synchronize()
    free_before = torch.cuda.mem_get_info(dev)[0]
    with torch.cuda.stream(stream):
        status = lib.mi355_w8a8_forward_static_ws_v1(ctypes.byref(p), int(stream.cuda_stream))
    stream.synchronize()
    assert status == 0
    assert torch.cuda.mem_get_info(dev)[0] == free_before
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    # captured: the library records kernel launches only (no allocation, no memset, no synchronisation)
    graph = torch.cuda.CUDAGraph()
    out.fill_(float("nan"))
    with torch.cuda.graph(graph, stream=stream):
        status = lib.mi355_w8a8_forward_static_ws_v1(ctypes.byref(p), int(torch.cuda.current_stream().cuda_stream))
    assert status == 0
    for _ in range(3):
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    assert torch.equal(first.view(torch.int16), want.view(torch.int16))


def test_static_workspace_refuses_to_keep_what_another_caller_may_have_overwritten(pkg):
    """The array is shared by every caller of the process: flags that tell a call to reuse an earlier call's
    packed operands or prologue are refused."""
    native = pkg._native
    lib = native.load()
    p = native.Problem()
    p.struct_size = ctypes.sizeof(p)
    p.m, p.k, p.n, p.n_adapters, p.rank = 64, 256, 256, 2, 8
    for flag in (native.FLAG_LORA_PACK_VALID, native.FLAG_SKIP_PROLOGUE):
        p.flags = flag
        assert lib.mi355_w8a8_forward_static_ws_v1(ctypes.byref(p), None) == -7  # MI355_W8A8_ERR_UNSUPPORTED


def test_static_workspace_rejects_what_does_not_fit(pkg):
    """A problem whose workspace exceeds the static array is refused on the host, before any launch."""
    native = pkg._native
    lib = native.load()
    m, k, n, n_ad, r = 8192, 4096, 24576, 8, 32
    assert lib.mi355_w8a8_workspace_bytes(m, k, n, n_ad, r, 1) > native.STATIC_WORKSPACE_BYTES
    p = native.Problem()
    p.struct_size = ctypes.sizeof(p)
    p.flags, p.m, p.k, p.n, p.n_adapters, p.rank = 1, m, k, n, n_ad, r
    assert lib.mi355_w8a8_forward_static_ws_v1(ctypes.byref(p), None) == -5  # MI355_W8A8_ERR_WORKSPACE
    assert lib.mi355_w8a8_forward_static_ws_v1(None, None) == -1
