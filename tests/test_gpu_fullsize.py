"""The benchmark configurations at full size: oracle comparison on row samples (rows are
independent units of this path) plus size-independent exact properties."""

import hashlib

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


def _sample_case(case, rows):
    sub = dict(case)
    sub["m"] = len(rows)
    sub["x"] = case["x"][rows]
    if "idx" in case:
        sub["idx"] = case["idx"][rows]
    if "residual" in case:
        sub["residual"] = case["residual"][rows]
    return sub


def _check_rows(case, got, aux, rows, what):
    st = wc.oracle_forward(_sample_case(case, rows), return_stages=True)
    if aux is not None:
        np.testing.assert_array_equal(aux["x_codes"][rows], st["x_codes"])
        np.testing.assert_array_equal(aux["x_scales"][rows].view(np.uint32), st["x_scales"].view(np.uint32))
        np.testing.assert_array_equal(aux["acc"][rows], st["acc"])
        if "normalized" in st:
            np.testing.assert_array_equal(o.bf16_bits(aux["normalized"][rows]), o.bf16_bits(st["normalized"]))
    rep = wc.compare(got[rows], st["out"])
    print(f"[parity-full]{what} {rep}", flush=True)
    # the reference gate's max-abs bound (0.25) presumes O(1) outputs; one bf16 ulp of a SwiGLU
    # product of magnitude 128 is already 1.0, so the elementwise tolerance is the bar here
    assert rep["violations"] == 0 and rep["relative_l2"] < 1e-2 and rep["cosine"] >= 0.9999, rep


def test_config2_full_size(dev):
    """Qwen3-8B gate/up, M4096 K4096 N24576, 8 adapters rank 32, RMSNorm + SwiGLU."""
    case = wc.make_case(4096, 4096, 24576, n_adapters=8, rank=32, seed=2, rms=True, swiglu=True)
    got, aux = wc.gpu_forward(case)
    rng = np.random.default_rng(0)
    rows = np.sort(rng.choice(4096, 160, replace=False))
    _check_rows(case, got, aux, rows, " cfg2")
    # rows are independent: permuting the rows of x (and of idx) permutes the output rows, bitwise
    perm = rng.permutation(4096)
    case_p = dict(case, x=case["x"][perm], idx=case["idx"][perm])
    got_p = wc.gpu_forward(case_p, return_aux=False)
    assert np.array_equal(o.bf16_bits(got_p), o.bf16_bits(got[perm]))
    # relabelling the adapters (permuting A, B, s and mapping idx) changes nothing, bitwise
    relabel = rng.permutation(8)
    inv = np.argsort(relabel)
    case_r = dict(case, a=case["a"][relabel], b=case["b"][relabel], s=case["s"][relabel],
                  idx=inv[case["idx"]].astype(np.int32))
    got_r = wc.gpu_forward(case_r, return_aux=False)
    assert np.array_equal(o.bf16_bits(got_r), o.bf16_bits(got))


def test_config2_base_is_linear_in_the_weight_scales(dev):
    """Doubling every per-channel scale doubles the pre-activation exactly (power-of-two scaling
    commutes with every float32 and bf16 rounding on the base path)."""
    case = wc.make_case(1024, 4096, 4096, n_adapters=0, seed=21)
    got = wc.gpu_forward(case, return_aux=False)
    case2 = dict(case, scales=case["scales"] * F32(2.0))
    got2 = wc.gpu_forward(case2, return_aux=False)
    assert np.array_equal(got2, got * F32(2.0))


@pytest.mark.parametrize("k,n", [(2560, 6144), (4096, 2560)])
def test_config4_m2048(dev, k, n):
    case = wc.make_case(2048, k, n, n_adapters=4, rank=64, alpha=128, seed=41, student_t=True)
    got, aux = wc.gpu_forward(case)
    rows = np.sort(np.random.default_rng(1).choice(2048, 128, replace=False))
    _check_rows(case, got, aux, rows, f" cfg4 m2048 {k}x{n}")


def test_config3_repeatable_and_row_permutation(dev):
    case = wc.make_case(16, 12288, 4096, n_adapters=16, rank=32, seed=3, residual=True, idx_mode="arange")
    a = wc.gpu_forward(case, return_aux=False)
    b = wc.gpu_forward(case, return_aux=False)
    assert hashlib.sha256(a.tobytes()).hexdigest() == hashlib.sha256(b.tobytes()).hexdigest()
    perm = np.random.default_rng(2).permutation(16)
    case_p = dict(case, x=case["x"][perm], idx=case["idx"][perm], residual=case["residual"][perm])
    c = wc.gpu_forward(case_p, return_aux=False)
    assert np.array_equal(o.bf16_bits(c), o.bf16_bits(a[perm]))


def test_config5_full_size_moe(dev):
    """Qwen3-30B-A3B-style expert MLP: 128 experts, top-8, T2048, hidden 2048, intermediate 768,
    rank-16 LoRA on every expert; ragged per-expert M from the routing histogram."""
    import torch

    from __graft_entry__ import load_package

    w8 = load_package().w8a8_lora
    rng = np.random.default_rng(wc.BASE_SEED + 5)
    t, h, inter, e, topk, r = 2048, 2048, 768, 128, 8, 16
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    logits = rng.standard_normal((t, e)).astype(F32)
    gu_codes = rng.integers(-127, 128, (e, h, 2 * inter), dtype=np.int8)
    gu_scales = rng.uniform(0.001, 0.01, (e, 2 * inter)).astype(F32)
    dn_codes = rng.integers(-127, 128, (e, inter, h), dtype=np.int8)
    dn_scales = rng.uniform(0.001, 0.01, (e, h)).astype(F32)
    mk = lambda shape: o.bf16_round((rng.standard_normal(shape) * 0.02).astype(F32))
    gua, gub, da, db = mk((e, h, r)), mk((e, r, 2 * inter)), mk((e, inter, r)), mk((e, r, h))
    gu = [o.GroupQuantizedWeight(gu_codes[i], gu_scales[i:i + 1], h, h, 8, h) for i in range(e)]
    dn = [o.GroupQuantizedWeight(dn_codes[i], dn_scales[i:i + 1], inter, inter, 8, inter) for i in range(e)]
    want, st = o.moe_expert_mlp(hidden, logits, topk, gu, dn, gua, gub, da, db, F32(1.0), return_stages=True)
    bf = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev).to(torch.bfloat16)
    guw = w8.prepare_grouped_weight(torch.from_numpy(gu_codes).to(dev), torch.from_numpy(gu_scales).to(dev))
    dnw = w8.prepare_grouped_weight(torch.from_numpy(dn_codes).to(dev), torch.from_numpy(dn_scales).to(dev))
    sizes = torch.from_numpy(st["group_sizes"].astype(np.int32))
    assert int(sizes.sum()) == t * topk and int(sizes.min()) >= 0

    # stage 1: grouped gate/up + SwiGLU on the oracle's sorted rows
    act_gpu = w8.grouped_forward(bf(st["x_sorted"]), sizes, guw, bf(gua), bf(gub), 1.0, swiglu=True)
    torch.cuda.synchronize()
    act_np = act_gpu.float().cpu().numpy()
    rep = wc.compare(act_np, st["act"])
    print(f"[parity-full] cfg5 gate_up+swiglu {rep}", flush=True)
    assert rep["violations"] == 0 and rep["relative_l2"] < 1e-2 and rep["cosine"] >= 0.9999, rep

    # stage 2: grouped down projection, oracle fed with the GPU's own stage-1 output (a one-ulp
    # difference upstream re-quantizes a whole row, so stages are compared one at a time)
    down_gpu = w8.grouped_forward(act_gpu, sizes, dnw, bf(da), bf(db), 1.0)
    torch.cuda.synchronize()
    down_want = o.bf16_round(o.grouped_quantized_lora_linear_f32(act_np, st["group_sizes"], dn, da, db, F32(1.0)))
    rep = wc.compare(down_gpu.float().cpu().numpy(), down_want)
    print(f"[parity-full] cfg5 down {rep}", flush=True)
    assert rep["violations"] == 0 and rep["relative_l2"] < 1e-2 and rep["cosine"] >= 0.9999, rep

    # end to end through the module-level composite (routing, both GEMMs, combine)
    got = w8.w8a8_moe_expert_mlp(bf(hidden), torch.from_numpy(logits).to(dev), topk, guw, dnw, bf(gua), bf(gub),
                                 bf(da), bf(db), 1.0, enabled=True)
    torch.cuda.synchronize()
    rep = wc.compare(got.float().cpu().numpy(), want)
    print(f"[parity-full] cfg5 end-to-end {rep}", flush=True)
    assert rep["relative_l2"] < 1e-3 and rep["cosine"] >= 0.9999 and rep["violations"] < 1e-3 * rep["size"], rep
