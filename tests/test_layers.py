"""Module-level mirror of the reference's LoRA layers (skyrl/tx/layers/lora.py).

The CPU half checks the host logic (fuse/split against the oracle, adapter initialisation,
validation, loud failure without a GPU).  The GPU half follows the reference's own closed-form
layer test (tests/tx/layers/test_lora_fast_path.py:17-49, 85-101, 207-239: ``arange`` parameters
divided by 97 / 89 / 53, scalings 0.25 / 0.75 / 1.25) with the geometry widened to K = 40 so the
rows fit the native path, and anchors the W8A8 numerics on the oracle.
"""

import numpy as np
import pytest

from oracle import w8a8_oracle as o
import w8a8_cases as wc

F32 = np.float32


@pytest.fixture(scope="module")
def pkg():
    from __graft_entry__ import load_package

    return load_package()


@pytest.fixture(scope="module")
def dev(pkg):
    torch = pytest.importorskip("torch")
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    pkg._native.load()
    return torch.device("cuda:0")


# --------------------------------------------------------------------------------------
# CPU: host logic
# --------------------------------------------------------------------------------------

@pytest.mark.parametrize("sizes", [(1, 1), (2, 1), (3, 5, 2), (4,)])
def test_fuse_and_split_match_the_oracle(pkg, sizes):
    import torch

    rng = np.random.default_rng(sum(sizes))
    groups = 6
    parts = [rng.standard_normal((2, 3, groups * g)).astype(F32) for g in sizes]
    fused = pkg.lora.FusedLoRALinear.fuse(*[torch.from_numpy(p) for p in parts], group_sizes=sizes)
    np.testing.assert_array_equal(fused.numpy(), o.fuse(*parts, group_sizes=sizes))
    back = pkg.lora.FusedLoRALinear.split(fused, sizes)
    want = o.split(fused.numpy(), sizes)
    assert len(back) == len(sizes)
    for got, ref, src in zip(back, want, parts):
        np.testing.assert_array_equal(got.numpy(), ref)
        np.testing.assert_array_equal(got.numpy(), src)


def test_fuse_places_group_members_side_by_side(pkg):
    """gate/up with group sizes (1, 1): columns alternate gate0, up0, gate1, up1, ..."""
    import torch

    gate = torch.arange(4.0).reshape(1, 4)
    up = torch.arange(4.0).reshape(1, 4) + 100
    fused = pkg.lora.FusedLoRALinear.fuse(gate, up, group_sizes=(1, 1))
    assert fused.tolist() == [[0, 100, 1, 101, 2, 102, 3, 103]]
    q, kv = torch.arange(6.0).reshape(1, 6), torch.arange(3.0).reshape(1, 3) + 50
    fused = pkg.lora.FusedLoRALinear.fuse(q, kv, group_sizes=(2, 1))
    assert fused.tolist() == [[0, 1, 50, 2, 3, 51, 4, 5, 52]]


def test_fuse_and_split_reject_bad_shapes(pkg):
    import torch

    F = pkg.lora.FusedLoRALinear
    with pytest.raises(ValueError):
        F.fuse(torch.zeros(2, 4), group_sizes=(1, 1))
    with pytest.raises(ValueError):
        F.fuse(torch.zeros(2, 4), torch.zeros(2, 5), group_sizes=(1, 1))
    with pytest.raises(ValueError):
        F.split(torch.zeros(2, 7), (1, 1))
    with pytest.raises(ValueError):
        F(8, 16, components=("gate", "up"), group_sizes=(1,), device="cpu")


def test_init_lora_adapter(pkg):
    import torch

    L = pkg.lora
    lin = L.LoRALinear(16, 8, max_lora_adapters=3, max_lora_rank=4, device="cpu")
    assert lin.lora_A.shape == (3, 16, 4) and lin.lora_B.shape == (3, 4, 8)
    assert torch.count_nonzero(lin.lora_A) == 0 and lin.lora_scaling.tolist() == [1, 1, 1]
    lin.lora_B[1] = 1
    L.init_lora_adapter(lin, 1, rank=2, alpha=8.0, seed=3)
    assert lin.lora_scaling.tolist() == [1, 4, 1] and lin.lora_ranks.tolist() == [4, 2, 4]
    a = lin.lora_A[1].float()
    assert torch.count_nonzero(a[:, :2]) == 32 and torch.count_nonzero(a[:, 2:]) == 0
    assert a.abs().max() <= (6.0 / 16) ** 0.5 + 1e-2
    assert torch.count_nonzero(lin.lora_B) == 0 and torch.count_nonzero(lin.lora_A[0]) == 0
    with pytest.raises(ValueError):
        L.init_lora_adapter(lin, 3, rank=2, alpha=1.0)
    with pytest.raises(ValueError):
        L.init_lora_adapter(lin, 0, rank=5, alpha=1.0)
    # expert layers divide the rank over the experts (lora.py:471-475)
    exp = L.LoRAExpert(4, 16, 8, max_lora_adapters=2, max_lora_rank=4, device="cpu")
    assert exp.lora_A.shape == (2, 4, 16, 4) and exp.lora_B.shape == (2, 4, 4, 8)
    L.init_lora_adapter(exp, 0, rank=8, alpha=16.0)
    assert exp.lora_ranks.tolist() == [2, 4] and exp.lora_scaling.tolist() == [8, 1]
    assert torch.count_nonzero(exp.lora_A[0, :, :, 2:]) == 0 and torch.count_nonzero(exp.lora_A[0, :, :, :2]) > 0
    # he_uniform counts the expert axis as receptive field (jax.nn.initializers, in_axis = -2):
    # fan_in = experts * in_features, so the bound is sqrt(6 / (4 * 16)), not sqrt(6 / 16)
    bound = (6.0 / (4 * 16)) ** 0.5
    amax = float(exp.lora_A[0].float().abs().max())
    assert amax <= bound * (1 + 2 ** -8) and amax > 0.8 * bound
    with pytest.raises(RuntimeError):
        L.init_lora_adapter(L.LoRALinear(16, 8, device="cpu"), 0, rank=2, alpha=1.0)


def test_constant_scaling_cache_survives_inference_mode(pkg):
    """A Python-float scaling first seen under inference_mode must still be usable by a later
    training call: the cached constant has to be an ordinary tensor that autograd can save."""
    import torch

    w8 = pkg.w8a8_lora
    with torch.inference_mode():
        first = w8._scaling_vector(0.3125, 1, torch.device("cpu"))
    assert not first.is_inference()
    s = w8._scaling_scalar(0.3125, torch.device("cpu"))
    assert s.data_ptr() == first.data_ptr()   # same cached constant on both paths

    class Keep(torch.autograd.Function):
        @staticmethod
        def forward(ctx, x, scaling):
            ctx.save_for_backward(x, scaling)
            return x * scaling

        @staticmethod
        def backward(ctx, g):
            x, scaling = ctx.saved_tensors
            return g * scaling, None

    x = torch.ones(3, requires_grad=True)
    Keep.apply(x, s).sum().backward()
    assert x.grad.tolist() == [0.3125] * 3


def test_layers_fail_loudly_without_a_gpu_path(pkg):
    import torch

    L, ql = pkg.lora, pkg.quantized_lora
    lin = L.LoRALinear(16, 8, max_lora_adapters=2, max_lora_rank=4, device="cpu")
    x = torch.zeros(1, 2, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="not loaded"):
        lin(x)
    lin.load_dense(torch.ones(16, 8))
    assert lin.weight.codes.dtype == torch.int8 and lin.weight.group_size == 16
    with pytest.raises(RuntimeError, match="GPU"):
        lin(x)                                     # CPU tensors: no CPU path
    with pytest.raises(RuntimeError, match="GPU"):
        lin(x, adapter_indices=torch.zeros(1, dtype=torch.int32))
    with pytest.raises(ValueError):
        lin.load_quantized(ql.quantize_frozen_weight(torch.ones(32, 8), bits=8, group_size=32))
    exp = L.LoRAExpert(2, 16, 8, max_lora_adapters=2, max_lora_rank=4, device="cpu")
    with pytest.raises(RuntimeError, match="not loaded"):
        exp(x[0], torch.tensor([1, 1]))
    with pytest.raises(RuntimeError, match="GPU"):
        exp.load_quantized(torch.zeros(2, 16, 8, dtype=torch.int8), torch.ones(2, 8))


def test_constant_lora_scalings_are_cached_per_value_count_and_device(pkg):
    """A Python-number ``lora_scaling`` must not become a host-to-device copy at every call."""
    import torch

    w8 = pkg.w8a8_lora
    a = w8._scaling_vector(2.5, 4, torch.device("cpu"))
    assert a.dtype == torch.float32 and a.tolist() == [2.5] * 4
    assert w8._scaling_vector(2.5, 4, torch.device("cpu")) is a          # the same tensor again
    assert w8._scaling_vector(2.5, 3, torch.device("cpu")).shape == (3,)
    assert w8._scaling_vector(2, 4, torch.device("cpu")) is not a
    t = torch.tensor([1.0, 2.0, 3.0])
    assert w8._scaling_vector(t, 3, torch.device("cpu")).tolist() == [1.0, 2.0, 3.0]   # tensors pass through
    assert w8._scaling_vector(torch.tensor(0.5), 2, torch.device("cpu")).tolist() == [0.5, 0.5]
    s = w8._scaling_scalar(0.25, torch.device("cpu"))
    assert s.ndim == 0 and float(s) == 0.25 and w8._scaling_scalar(t, torch.device("cpu")) is t


# --------------------------------------------------------------------------------------
# GPU: the layers through the HIP path
# --------------------------------------------------------------------------------------

K_IN, N_OUT, RANK, N_AD = 40, 7, 3, 3


def _closed_form_layer(pkg, dev, cls=None, n_out=None, **kw):
    import torch

    L = pkg.lora
    cls = cls or L.LoRALinear
    n_out = n_out or N_OUT
    layer = cls(K_IN, n_out, max_lora_adapters=N_AD, max_lora_rank=RANK, device=dev, **kw)
    kernel = o.bf16_round((np.arange(K_IN * n_out, dtype=F32).reshape(K_IN, n_out) / 53.0) % 3.0 - 1.5)
    a = o.bf16_round(np.arange(N_AD * K_IN * RANK, dtype=F32).reshape(N_AD, K_IN, RANK) / 97.0 / 8.0)
    b = o.bf16_round(np.arange(N_AD * RANK * n_out, dtype=F32).reshape(N_AD, RANK, n_out) / 89.0)
    s = np.asarray([0.25, 0.75, 1.25], dtype=F32)
    layer.load_dense(torch.from_numpy(kernel))
    layer.lora_A = torch.from_numpy(a).to(dev).to(torch.bfloat16)
    layer.lora_B = torch.from_numpy(b).to(dev).to(torch.bfloat16)
    layer.lora_scaling = torch.from_numpy(s).to(dev)
    w = o.quantize_frozen_weight(kernel, bits=8, group_size=K_IN, scale_dtype="f32")
    np.testing.assert_array_equal(layer.weight.codes.cpu().numpy(), w.codes)
    return layer, kernel, w, a, b, s


def _to_np(t):
    import torch

    torch.cuda.synchronize()
    return t.to(torch.float32).cpu().numpy()


@pytest.mark.gpu
def test_linear_single_adapter_matches_direct_formula(pkg, dev):
    import torch

    layer, kernel, w, a, b, s = _closed_form_layer(pkg, dev)
    x = o.bf16_round(np.arange(4 * K_IN, dtype=F32).reshape(1, 4, K_IN) / 19.0 / 8.0)
    xt = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    for adapter in (0, 2):
        got = _to_np(layer(xt, adapter_indices=torch.tensor([adapter], dtype=torch.int32, device=dev)))
        assert got.shape == (1, 4, N_OUT)
        want = o.quantized_lora_linear(x[0], w, a[adapter], b[adapter], s[adapter])
        rep = wc.compare(got[0], want)
        assert rep["violations"] == 0, rep
        # the reference's float formula, to the gate the reference sets for W8A8 against dense
        direct = x[0] @ kernel + (x[0] @ a[adapter]) @ b[adapter] * s[adapter]
        gate = o.numerical_gate(got[0], direct)
        assert gate["relative_l2"] < 1e-2 and gate["cosine"] >= 0.9999, gate
    # no adapter indices: base only (lora.py:129-130)
    base = _to_np(layer(xt))
    assert wc.compare(base[0], o.quantized_frozen_linear(x[0], w))["violations"] == 0
    assert np.abs(base - got).max() > 0.1


@pytest.mark.gpu
def test_linear_routes_one_adapter_per_example(pkg, dev):
    import torch

    layer, kernel, w, a, b, s = _closed_form_layer(pkg, dev)
    x = o.bf16_round(np.arange(2 * 4 * K_IN, dtype=F32).reshape(2, 4, K_IN) / 37.0 / 8.0)
    xt = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    got = _to_np(layer(xt, adapter_indices=torch.tensor([0, 2], dtype=torch.int32, device=dev)))
    assert got.shape == (2, 4, N_OUT)
    for example, adapter in enumerate((0, 2)):
        want = o.quantized_lora_linear(x[example], w, a[adapter], b[adapter], s[adapter])
        assert wc.compare(got[example], want)["violations"] == 0
        other = o.quantized_lora_linear(x[example], w, a[1], b[1], s[1])
        assert wc.compare(got[example], other)["violations"] > 0
    with pytest.raises(ValueError):
        layer(xt, adapter_indices=torch.tensor([0, 1, 2], dtype=torch.int32, device=dev))


@pytest.mark.gpu
def test_fused_linear_returns_one_tensor_per_component(pkg, dev):
    import torch

    L = pkg.lora
    k, n_each, r = 64, 24, 4
    rng = np.random.default_rng(11)
    gate, up = (o.bf16_round(rng.standard_normal((k, n_each)).astype(F32) * 0.1) for _ in range(2))
    fused_kernel = o.fuse(gate, up, group_sizes=(1, 1))
    layer = L.FusedLoRALinear(k, 2 * n_each, components=("gate_proj", "up_proj"), group_sizes=(1, 1),
                              max_lora_adapters=2, max_lora_rank=r, device=dev)
    layer.load_dense(torch.from_numpy(fused_kernel))
    a = o.bf16_round(rng.standard_normal((2, k, r)).astype(F32) * 0.1)
    b = o.bf16_round(rng.standard_normal((2, r, 2 * n_each)).astype(F32) * 0.1)
    layer.lora_A = torch.from_numpy(a).to(dev).to(torch.bfloat16)
    layer.lora_B = torch.from_numpy(b).to(dev).to(torch.bfloat16)
    layer.lora_scaling = torch.tensor([0.5, 2.0], device=dev)
    x = o.bf16_round(rng.standard_normal((3, 5, k)).astype(F32))
    idx = np.asarray([1, 0, 1], dtype=np.int32)
    out = layer(torch.from_numpy(x).to(dev).to(torch.bfloat16), torch.from_numpy(idx).to(dev))
    assert isinstance(out, tuple) and len(out) == 2
    w = o.quantize_frozen_weight(fused_kernel, bits=8, group_size=k, scale_dtype="f32")
    want = o.quantized_lora_linear_multi(x.reshape(15, k), w, a, b, np.asarray([0.5, 2.0], F32),
                                         np.repeat(idx, 5)).reshape(3, 5, 2 * n_each)
    want_gate, want_up = o.split(want, (1, 1))
    assert out[0].shape == (3, 5, n_each)
    assert wc.compare(_to_np(out[0]), want_gate)["violations"] == 0
    assert wc.compare(_to_np(out[1]), want_up)["violations"] == 0


@pytest.mark.gpu
def test_expert_layer_uses_expert_major_adapter_pairs(pkg, dev):
    """LoRA pair of a row = (its expert, its adapter), flattened expert * max_adapters + adapter
    (lora.py:414-431); rows keep their order."""
    import torch

    L = pkg.lora
    n_exp, n_ad, k, n, r = 4, 3, 64, 48, 4
    rng = np.random.default_rng(5)
    layer = L.LoRAExpert(n_exp, k, n, max_lora_adapters=n_ad, max_lora_rank=r, device=dev)
    dense = o.bf16_round(rng.standard_normal((n_exp, k, n)).astype(F32) * 0.1)
    ws = [o.quantize_frozen_weight(dense[e], bits=8, group_size=k, scale_dtype="f32") for e in range(n_exp)]
    codes = np.stack([w.codes for w in ws])
    scales = np.stack([np.asarray(w.scales, F32).reshape(n) for w in ws])
    layer.load_quantized(torch.from_numpy(codes), torch.from_numpy(scales))
    a = o.bf16_round(rng.standard_normal((n_ad, n_exp, k, r)).astype(F32) * 0.1)
    b = o.bf16_round(rng.standard_normal((n_ad, n_exp, r, n)).astype(F32) * 0.1)
    s = np.asarray([0.25, 0.75, 1.25], dtype=F32)
    layer.lora_A = torch.from_numpy(a).to(dev).to(torch.bfloat16)
    layer.lora_B = torch.from_numpy(b).to(dev).to(torch.bfloat16)
    layer.lora_scaling = torch.from_numpy(s).to(dev)
    group_sizes = np.asarray([13, 0, 21, 16], dtype=np.int32)   # one empty expert
    rows = int(group_sizes.sum())
    expert = np.repeat(np.arange(n_exp), group_sizes)
    adapter = rng.integers(0, n_ad, rows).astype(np.int32)
    x = o.bf16_round(rng.standard_normal((rows, k)).astype(F32))
    xt = torch.from_numpy(x).to(dev).to(torch.bfloat16)
    got = _to_np(layer(xt, torch.from_numpy(group_sizes).to(dev), torch.from_numpy(adapter).to(dev),
                       group_offset=torch.zeros(1, dtype=torch.int32)))
    want = np.stack([o.quantized_lora_linear(x[i:i + 1], ws[expert[i]], a[adapter[i], expert[i]],
                                             b[adapter[i], expert[i]], s[adapter[i]])[0] for i in range(rows)])
    rep = wc.compare(got, want)
    assert rep["violations"] == 0, rep
    # base only without adapter indices
    base = _to_np(layer(xt, torch.from_numpy(group_sizes).to(dev)))
    want_base = np.stack([o.quantized_frozen_linear(x[i:i + 1], ws[expert[i]])[0] for i in range(rows)])
    assert wc.compare(base, want_base)["violations"] == 0
    # swapping two adapters' parameters and the indices that name them changes nothing
    layer.lora_A = layer.lora_A[[1, 0, 2]].contiguous()
    layer.lora_B = layer.lora_B[[1, 0, 2]].contiguous()
    layer.lora_scaling = layer.lora_scaling[[1, 0, 2]].contiguous()
    swapped = np.where(adapter == 0, 1, np.where(adapter == 1, 0, adapter)).astype(np.int32)
    again = _to_np(layer(xt, torch.from_numpy(group_sizes).to(dev), torch.from_numpy(swapped).to(dev)))
    np.testing.assert_array_equal(again, got)
    # rows beyond sum(group_sizes) belong to no expert: zeros, and the rows in use do not move;
    # an adapter index outside the table is clamped like the kernels clamp it
    spare = 5
    x_long = torch.cat([xt, torch.ones(spare, k, dtype=torch.bfloat16, device=dev)])
    idx_long = torch.cat([torch.from_numpy(swapped), torch.full((spare,), 99, dtype=torch.int32)]).to(dev)
    longer = _to_np(layer(x_long, torch.from_numpy(group_sizes).to(dev), idx_long))
    np.testing.assert_array_equal(longer[:rows], got)
    assert not longer[rows:].any()
    with pytest.raises(NotImplementedError):
        layer(xt, torch.from_numpy(group_sizes).to(dev), group_offset=torch.ones(1, dtype=torch.int32))


@pytest.mark.gpu
def test_linear_gradients_match_oracle_and_generic_routing(pkg, dev):
    """The reference's gradient test (tests/tx/layers/test_lora_fast_path.py:103-133): the loss on the
    first example must give the same gradients whether the batch holds that example alone or a
    second one behind it; here the values are also checked against the oracle's backward."""
    import torch

    n_out = 8  # the native backward takes output widths that are multiples of 8
    layer, kernel, w, a, b, s = _closed_form_layer(pkg, dev, n_out=n_out)
    x = o.bf16_round(np.arange(4 * K_IN, dtype=F32).reshape(1, 4, K_IN) / 17.0 / 8.0)
    cot = o.bf16_round(np.arange(4 * n_out, dtype=F32).reshape(4, n_out) / 31.0)
    cot_t = torch.from_numpy(cot).to(dev)

    def grads(duplicate):
        for name in ("lora_A", "lora_B", "lora_scaling"):
            setattr(layer, name, getattr(layer, name).detach().clone().requires_grad_(True))
        xt = torch.from_numpy(x).to(dev).to(torch.bfloat16).requires_grad_(True)
        inp, indices = xt, torch.tensor([1], dtype=torch.int32, device=dev)
        if duplicate:
            inp = torch.cat([xt, (xt * 0.5 + 0.25).detach()], dim=0)
            indices = torch.tensor([1, 1], dtype=torch.int32, device=dev)
        out = layer(inp, adapter_indices=indices)[0]
        loss = (out.float() * cot_t).sum()
        loss.backward()
        torch.cuda.synchronize()
        f = lambda t: t.grad.detach().float().cpu().numpy()
        return float(loss.detach()), f(xt), f(layer.lora_A), f(layer.lora_B), f(layer.lora_scaling)

    fast, generic = grads(False), grads(True)
    assert abs(fast[0] - generic[0]) <= 2e-2 * max(1.0, abs(fast[0]))
    np.testing.assert_array_equal(fast[1], generic[1])           # dx of the first example: same rows, same kernels
    want = o.quantized_lora_linear_bwd(x[0], w, a[1], b[1], s[1], cot, relaxed_weight=True)
    assert wc.compare(fast[1][0], want[0])["violations"] == 0
    assert wc.compare(fast[2][1], want[1])["violations"] == 0
    assert wc.compare(fast[3][1], want[2])["violations"] == 0
    np.testing.assert_allclose(fast[4][1], want[3], rtol=1e-3)
    # adapters no row names receive zero gradients
    assert not fast[2][[0, 2]].any() and not fast[3][[0, 2]].any() and not fast[4][[0, 2]].any()
    # the duplicated batch adds the second example's rows to the LoRA gradients only through the
    # loss, which ignores them: same values up to the summation order
    for i in (2, 3):
        assert wc.compare(generic[i], fast[i])["violations"] == 0


@pytest.mark.gpu
def test_expert_layer_gradients_match_oracle(pkg, dev):
    """Gradients of the expert layer: per expert, the oracle's multi-adapter backward over that
    expert's rows; the scaling gradient adds up over the experts that share an adapter."""
    import torch

    L = pkg.lora
    n_exp, n_ad, k, n, r = 3, 2, 64, 48, 4
    rng = np.random.default_rng(8)
    layer = L.LoRAExpert(n_exp, k, n, max_lora_adapters=n_ad, max_lora_rank=r, device=dev)
    dense = o.bf16_round(rng.standard_normal((n_exp, k, n)).astype(F32) * 0.1)
    ws = [o.quantize_frozen_weight(dense[e], bits=8, group_size=k, scale_dtype="f32") for e in range(n_exp)]
    layer.load_quantized(torch.from_numpy(np.stack([w.codes for w in ws])),
                         torch.from_numpy(np.stack([np.asarray(w.scales, F32).reshape(n) for w in ws])))
    a = o.bf16_round(rng.standard_normal((n_ad, n_exp, k, r)).astype(F32) * 0.1)
    b = o.bf16_round(rng.standard_normal((n_ad, n_exp, r, n)).astype(F32) * 0.1)
    s = np.asarray([0.5, 1.5], dtype=F32)
    layer.lora_A = torch.from_numpy(a).to(dev).to(torch.bfloat16).requires_grad_(True)
    layer.lora_B = torch.from_numpy(b).to(dev).to(torch.bfloat16).requires_grad_(True)
    layer.lora_scaling = torch.from_numpy(s).to(dev).requires_grad_(True)
    group_sizes = np.asarray([17, 0, 30], dtype=np.int32)
    rows = int(group_sizes.sum())
    expert = np.repeat(np.arange(n_exp), group_sizes)
    adapter = rng.integers(0, n_ad, rows).astype(np.int32)
    x = o.bf16_round(rng.standard_normal((rows, k)).astype(F32))
    cot = o.bf16_round(rng.standard_normal((rows, n)).astype(F32))
    xt = torch.from_numpy(x).to(dev).to(torch.bfloat16).requires_grad_(True)
    out = layer(xt, torch.from_numpy(group_sizes).to(dev), torch.from_numpy(adapter).to(dev))
    (out.float() * torch.from_numpy(cot).to(dev)).sum().backward()
    torch.cuda.synchronize()
    f = lambda t: t.grad.detach().float().cpu().numpy()
    dx, da, db, ds = f(xt), f(layer.lora_A), f(layer.lora_B), f(layer.lora_scaling)
    want_ds = np.zeros(n_ad, dtype=np.float64)
    for e in range(n_exp):
        sel = np.nonzero(expert == e)[0]
        if sel.size == 0:
            assert not da[:, e].any() and not db[:, e].any()
            continue
        want = o.quantized_lora_linear_multi_bwd(x[sel], ws[e], a[:, e], b[:, e], s, adapter[sel], cot[sel],
                                                 relaxed_weight=True)
        assert wc.compare(dx[sel], want[0])["violations"] == 0
        assert wc.compare(da[:, e], want[1])["violations"] == 0
        assert wc.compare(db[:, e], want[2])["violations"] == 0
        want_ds += want[3]
    np.testing.assert_allclose(ds, want_ds, rtol=2e-3, atol=1e-3)


def test_fused_checkpoint_loading(pkg):
    """Component kernels and split adapters land in the fused layout of the reference's loader
    (skyrl/tx/utils/models.py:149-191): interleaved by group, quantized per output channel."""
    import torch

    L = pkg.lora
    rng = np.random.default_rng(4)
    k, heads, hd = 16, 2, 4                       # q has 2 heads per kv head
    q = rng.standard_normal((k, heads * 2 * hd)).astype(F32)
    kk = rng.standard_normal((k, heads * hd)).astype(F32)
    v = rng.standard_normal((k, heads * hd)).astype(F32)
    sizes = (2 * hd, hd, hd)
    layer = L.FusedLoRALinear(k, q.shape[1] + kk.shape[1] + v.shape[1], components=("q_proj", "k_proj", "v_proj"),
                              group_sizes=sizes, max_lora_adapters=2, max_lora_rank=4, device="cpu")
    layer.load_components([torch.from_numpy(t) for t in (q, kk, v)])
    want = o.quantize_frozen_weight(o.fuse(q, kk, v, group_sizes=sizes), bits=8, group_size=k, scale_dtype="f32")
    np.testing.assert_array_equal(layer.weight.codes.numpy(), want.codes)
    np.testing.assert_array_equal(layer.weight.scales.numpy(), want.scales)
    a = torch.from_numpy(rng.standard_normal((k, 4)).astype(F32))
    bs = [torch.from_numpy(rng.standard_normal((4, t.shape[1])).astype(F32)) for t in (q, kk, v)]
    layer.load_split_adapter(1, [a, a.clone(), a.clone()], bs)
    np.testing.assert_array_equal(layer.lora_B[1].float().numpy(),
                                  o.bf16_round(o.fuse(*[b.numpy() for b in bs], group_sizes=sizes)))
    np.testing.assert_array_equal(layer.lora_A[1].float().numpy(), o.bf16_round(a.numpy()))
    assert not layer.lora_A[0].any()
    with pytest.raises(RuntimeError, match="share the same lora_A"):
        layer.load_split_adapter(0, [a, a + 1, a], bs)
    with pytest.raises(ValueError):
        layer.load_components([torch.from_numpy(q)])


def test_version_counter_is_optional(pkg):
    """``_version_of`` reads a tensor's version counter and answers None for tensors torch keeps none for
    (made under ``torch.inference_mode()``), which the plans then treat as written at every run."""
    import torch

    w8 = pkg.w8a8_lora
    t = torch.ones(3)
    v0 = w8._version_of(t)
    t.add_(1.0)
    assert isinstance(v0, int) and w8._version_of(t) == v0 + 1
    with torch.inference_mode():
        u = torch.ones(3)
    assert w8._version_of(u) is None
