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
