"""GPU parity of the group-scaled quantized linear (W4 / W8 codes, A4 / A8 activations, scales per K
group) through the C ABI, against the CPU oracle and the reference's hand-coded W4A4 case.

Bar: activation codes and scales bit for bit; above 32 rows also the float32 base (the sum over
the groups before the LoRA term) and, without LoRA, the bf16 output; otherwise |a - b| <= 2e-2 +
1e-2 |b| (the float32 summation order of the LoRA products differs, and the decode kernel for up to
32 rows adds the groups per wave before it adds the waves).
"""

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


def _to_dev(pkg, dev, w):
    import torch

    return pkg.quantized_lora.GroupQuantizedWeight(torch.from_numpy(w.codes).to(dev), torch.from_numpy(w.scales).to(dev),
                                                   w.original_in_features, w.padded_in_features, w.bits, w.group_size)


def _bf(dev, v):
    import torch

    return torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(torch.bfloat16)


def test_reference_hand_coded_w4a4_case(dev, pkg):
    """tests/tx/kernels/test_quantized_lora.py:58-74 (groups of 2) embedded in groups of 32: every
    group is followed by 30 zero weights and zero activations, which changes no amax, code or sum."""
    import torch

    small = o.GroupQuantizedWeight(codes=np.asarray([[0x31, 0x4E], [0x0B, 0x96]], dtype=np.uint8),
                                   scales=np.asarray([[0.5, 2.0], [1.5, 0.25]], dtype=F32), original_in_features=3,
                                   padded_in_features=4, bits=4, group_size=2)
    x_small = np.asarray([[7.0, -3.0, -7.0], [0.0, 0.0, 3.0]], dtype=F32)
    expected = np.asarray([[51.5, -62.5], [-22.5, 4.5]], dtype=F32)
    np.testing.assert_allclose(o.quantized_frozen_linear_f32(x_small, small, activation_bits=4), expected, rtol=1e-6)
    codes = np.zeros((64, 2), dtype=np.int8)
    codes[[0, 1, 32, 33]] = o.unpack_signed_int4(small.codes)
    x = np.zeros((2, 64), dtype=F32)
    x[:, [0, 1, 32]] = x_small
    big = o.GroupQuantizedWeight(codes=o.pack_signed_int4(codes), scales=small.scales, original_in_features=64,
                                 padded_in_features=64, bits=4, group_size=32)
    got, aux = pkg.gq_linear.forward(_bf(dev, x), _to_dev(pkg, dev, big), activation_bits=4, return_aux=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(aux["base"].cpu().numpy(), expected)
    np.testing.assert_array_equal(got.to(torch.float32).cpu().numpy(), expected)
    via_api = pkg.quantized_lora.quantized_frozen_linear(_bf(dev, x), _to_dev(pkg, dev, big), activation_bits=4)
    assert torch.equal(via_api, got)
    # and the reference's own weight (groups of 2, K = 3 padded to 4) straight through the entry point, which
    # embeds it the same way by itself
    direct = pkg.quantized_lora.quantized_frozen_linear(_bf(dev, x_small), _to_dev(pkg, dev, small), activation_bits=4)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(direct.to(torch.float32).cpu().numpy(), expected)


def test_per_channel_w8a8_with_k_not_a_multiple_of_8(dev, pkg):
    """quantized_lora_linear (quantized_lora.py:257-304) takes any K: a per-channel W8A8 weight with K = 100
    runs as one group of 128 on the group-scaled kernels, codes, scales and float32 base bit-equal to the oracle."""
    import torch

    rng = np.random.default_rng(100)
    m, k, n, r = 40, 100, 72, 8
    x = o.bf16_round(rng.standard_t(4, (m, k)).astype(F32))
    w = o.quantize_frozen_weight((rng.standard_normal((k, n)) * 0.05).astype(F32), bits=8, group_size=k, scale_dtype="f32")
    a = o.bf16_round((rng.standard_normal((k, r)) * 0.05).astype(F32))
    b = o.bf16_round((rng.standard_normal((r, n)) * 0.05).astype(F32))
    base = o.quantized_frozen_linear_f32(x, w, activation_bits=8)
    want = o.bf16_round((base + o.lora_delta_multi(x, a[None], b[None], np.asarray([1.5], F32), np.zeros(m, np.int32))).astype(F32))
    got = pkg.quantized_lora.quantized_lora_linear(_bf(dev, x), _to_dev(pkg, dev, w), _bf(dev, a), _bf(dev, b), 1.5)
    frozen = pkg.quantized_lora.quantized_frozen_linear(_bf(dev, x), _to_dev(pkg, dev, w))
    torch.cuda.synchronize()
    np.testing.assert_array_equal(o.bf16_bits(frozen.to(torch.float32).cpu().numpy()), o.bf16_bits(o.bf16_round(base)))
    rep = wc.compare(got.to(torch.float32).cpu().numpy(), want)
    assert rep["violations"] == 0, rep


CASES = [
    # m, k, n, weight bits, activation bits, group, rank, adapters
    (5, 64, 17, 4, 8, 32, 0, 0),
    (33, 200, 96, 4, 4, 64, 8, 1),        # K padded to 256
    (70, 512, 264, 8, 8, 128, 16, 3),     # W8 with grouped scales, three adapters
    (16, 1024, 520, 4, 8, 64, 32, 4),
    (128, 384, 130, 8, 4, 96, 0, 0),      # group of three k blocks, A4
    (300, 2048, 256, 4, 8, 2048, 64, 2),  # one group: per-channel W4
    (45, 100, 40, 4, 8, 32, 5, 3),        # K not a multiple of 8: LoRA-A by the wave-per-row kernel
    (90, 256, 72, 8, 8, 64, 12, 1),       # one adapter without indices
    (2050, 200, 2056, 4, 8, 64, 8, 3),    # many tiles, ragged edges, an odd number of k blocks
    (2048, 384, 2048, 8, 4, 96, 0, 0),    # 8-bit codes, three k blocks a group
    (1024, 2048, 512, 4, 8, 1024, 40, 5),  # long groups
    (260, 256, 136, 4, 8, 64, 24, 20),    # twenty adapters: three batches of the LDS-staged LoRA epilogue
    (130, 128, 132, 8, 8, 64, 8, 3),      # N not a multiple of 8: the epilogue that reads B from memory
    (33, 200, 96, 4, 8, 50, 8, 2),        # groups of 50: embedded in groups of 64 with zero codes behind every group
    (20, 36, 40, 4, 4, 2, 0, 0),          # the reference test's group size: groups of 2 in groups of 32
    (64, 100, 48, 8, 8, 100, 6, 1),       # per-channel W8A8 with K = 100: one group of 128
    (70, 90, 56, 8, 4, 30, 12, 3),        # K padded to the group (90 -> 3 x 30), groups of 30
]


@pytest.mark.parametrize("m,k,n,wb,ab,group,rank,n_ad", CASES)
def test_gq_linear_matches_oracle(dev, pkg, m, k, n, wb, ab, group, rank, n_ad):
    import torch

    rng = np.random.default_rng(m * 7 + k + n)
    x = o.bf16_round(rng.standard_t(4, (m, k)).astype(F32))
    w = o.quantize_frozen_weight((rng.standard_normal((k, n)) * 0.05).astype(F32), bits=wb, group_size=group,
                                 scale_dtype="f32")
    print(f"[case] gq linear m={m} k={k} n={n} W{wb}A{ab} group={group} rank={rank} adapters={n_ad}", flush=True)
    base, x_codes, x_scales, _ = o.quantized_frozen_linear_f32(x, w, activation_bits=ab, return_parts=True)
    a = b = s = idx = None
    want_f32 = base
    if n_ad:
        a = o.bf16_round((rng.standard_normal((n_ad, k, rank)) * 0.05).astype(F32))
        b = o.bf16_round((rng.standard_normal((n_ad, rank, n)) * 0.05).astype(F32))
        s = rng.uniform(0.5, 2.0, n_ad).astype(F32)
        idx = rng.integers(0, n_ad, m).astype(np.int32)
        want_f32 = (base + o.lora_delta_multi(x, a, b, s, idx)).astype(F32)
        if n_ad == 1:
            idx = None                # no indices: every row takes adapter 0
    got, aux = pkg.gq_linear.forward(_bf(dev, x), _to_dev(pkg, dev, w), None if a is None else _bf(dev, a),
                                     None if b is None else _bf(dev, b),
                                     None if s is None else torch.from_numpy(s).to(dev), activation_bits=ab,
                                     adapter_indices=None if idx is None else torch.from_numpy(idx).to(dev),
                                     return_aux=True)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(aux["x_codes"].cpu().numpy(), x_codes.reshape(m, -1))
    np.testing.assert_array_equal(aux["x_scales"].cpu().numpy().view(np.uint32), x_scales.view(np.uint32))
    if m > 32:
        np.testing.assert_array_equal(aux["base"].cpu().numpy().view(np.uint32), base.view(np.uint32))
    else:   # decode kernel: the groups are summed per wave, then the waves (same terms, other order)
        np.testing.assert_allclose(aux["base"].cpu().numpy(), base, rtol=2e-6, atol=1e-6 * float(np.abs(base).max()))
    got_np = got.to(torch.float32).cpu().numpy()
    want = o.bf16_round(want_f32)
    if not n_ad and m > 32:
        np.testing.assert_array_equal(o.bf16_bits(got_np), o.bf16_bits(want))
    rep = wc.compare(got_np, want)
    print(f"[gq parity] m{m}k{k}n{n} W{wb}A{ab} {rep}", flush=True)
    assert rep["violations"] == 0, rep


@pytest.mark.parametrize("m,k,n,wb,ab,group,rank,n_ad", [
    (70, 512, 264, 8, 8, 128, 16, 3),
    (2050, 200, 2056, 4, 8, 64, 8, 3),     # ragged edges in both directions
    (333, 1024, 1100, 4, 4, 256, 0, 0),
    (260, 256, 136, 4, 8, 64, 24, 20),     # more adapters than one batch of the staged LoRA epilogue holds
    (130, 128, 132, 8, 8, 64, 8, 3),       # N not a multiple of 8
])
def test_gq_lds_staged_and_direct_kernels_agree_bitwise(dev, pkg, m, k, n, wb, ab, group, rank, n_ad):
    """Groups of whole 64-wide k steps run on the LDS-staged 128 x 128 tiles; the kernel that feeds its wave
    tiles from the L2 (FLAG_GQ_DIRECT) gives the same float32 base and the same output, bit for bit."""
    import torch

    rng = np.random.default_rng(m + 3 * k + 5 * n)
    x = o.bf16_round(rng.standard_t(4, (m, k)).astype(F32))
    w = o.quantize_frozen_weight((rng.standard_normal((k, n)) * 0.05).astype(F32), bits=wb, group_size=group,
                                 scale_dtype="f32")
    args = [_bf(dev, x), _to_dev(pkg, dev, w)]
    kw = dict(activation_bits=ab, return_aux=True)
    if n_ad:
        a = o.bf16_round((rng.standard_normal((n_ad, k, rank)) * 0.05).astype(F32))
        b = o.bf16_round((rng.standard_normal((n_ad, rank, n)) * 0.05).astype(F32))
        args += [_bf(dev, a), _bf(dev, b), torch.from_numpy(rng.uniform(0.5, 2.0, n_ad).astype(F32)).to(dev)]
        kw["adapter_indices"] = torch.from_numpy(rng.integers(0, n_ad, m).astype(np.int32)).to(dev)
    print(f"[case] gq kernels m={m} k={k} n={n} W{wb}A{ab} group={group}", flush=True)
    staged, aux_s = pkg.gq_linear.forward(*args, **kw)
    direct, aux_d = pkg.gq_linear.forward(*args, flags=pkg._native.FLAG_GQ_DIRECT, **kw)
    torch.cuda.synchronize()
    assert torch.equal(aux_s["base"].view(torch.int32), aux_d["base"].view(torch.int32))
    assert torch.equal(staged.view(torch.int16), direct.view(torch.int16))


def test_gq_single_adapter_through_the_reference_entry_point(dev, pkg):
    import torch

    rng = np.random.default_rng(9)
    m, k, n, r = 24, 256, 64, 8
    x = o.bf16_round(rng.standard_normal((2, m // 2, k)).astype(F32))
    w = o.quantize_frozen_weight(rng.standard_normal((k, n)).astype(F32) * 0.1, bits=4, group_size=64)   # bf16 scales
    a = o.bf16_round((rng.standard_normal((k, r)) * 0.1).astype(F32))
    b = o.bf16_round((rng.standard_normal((r, n)) * 0.1).astype(F32))
    want = o.quantized_lora_linear(x, w, a, b, F32(0.75), activation_bits=8)
    import torch as _t
    wt = pkg.quantized_lora.GroupQuantizedWeight(_t.from_numpy(w.codes).to(dev),
                                                 _t.from_numpy(w.scales).to(dev).to(_t.bfloat16), k, k, 4, 64)
    got = pkg.quantized_lora.quantized_lora_linear(_bf(dev, x), wt, _bf(dev, a), _bf(dev, b), 0.75)
    torch.cuda.synchronize()
    assert tuple(got.shape) == (2, m // 2, n)
    rep = wc.compare(got.to(torch.float32).cpu().numpy(), want)
    assert rep["violations"] == 0, rep


def test_gq_pack_keeps_four_bits_and_rejects_bad_geometry(dev, pkg):
    import torch

    lib = pkg._native.load()
    assert lib.mi355_w8a8_gq_packed_weight_bytes(64, 32, 4) == 2 * 512
    assert lib.mi355_w8a8_gq_packed_weight_bytes(64, 33, 8) == 2 * 2 * 1024
    assert lib.mi355_w8a8_gq_packed_weight_bytes(48, 32, 4) == 0
    assert lib.mi355_w8a8_gq_workspace_bytes(4, 64, 10, 0, 0) == 0
    assert lib.mi355_w8a8_gq_workspace_bytes(4, 64, 32, 2, 8) > lib.mi355_w8a8_gq_workspace_bytes(4, 64, 32, 0, 0) > 0
    w = o.quantize_frozen_weight(np.ones((70, 8), F32), bits=4, group_size=14, scale_dtype="f32")
    # (the C entry points take groups of whole 32-wide k blocks only -- the workspace query above says so; the
    # host mirror embeds other group sizes, here 14 in 32)
    ones = pkg.gq_linear.forward(torch.ones(2, 70, dtype=torch.bfloat16, device=dev), _to_dev(pkg, dev, w))
    want = o.bf16_round(o.quantized_frozen_linear_f32(np.ones((2, 70), F32), w, activation_bits=8))
    np.testing.assert_array_equal(ones.to(torch.float32).cpu().numpy(), want)
    w = o.quantize_frozen_weight(np.ones((64, 8), F32), bits=4, group_size=32, scale_dtype="f32")
    wt = _to_dev(pkg, dev, w)
    with pytest.raises(ValueError):
        pkg.gq_linear.forward(torch.zeros(2, 60, dtype=torch.bfloat16, device=dev), wt)
    with pytest.raises(TypeError):
        pkg.gq_linear.forward(torch.zeros(2, 64, dtype=torch.float32, device=dev), wt)
    with pytest.raises(ValueError):
        pkg.gq_linear.forward(torch.zeros(2, 64, dtype=torch.bfloat16, device=dev), wt, activation_bits=5)
    with pytest.raises(ValueError):
        pkg.gq_linear.forward(torch.zeros(2, 64, dtype=torch.bfloat16, device=dev), wt,
                              adapter_indices=torch.zeros(2, dtype=torch.int32, device=dev))


@pytest.mark.parametrize("m,k,n,wb,ab,group,rank", [(70, 256, 96, 4, 8, 64, 8), (33, 200, 48, 8, 4, 50, 5)])
def test_group_scaled_lora_linear_under_autograd(dev, pkg, m, k, n, wb, ab, group, rank):
    """quantized_lora_linear on a group-scaled geometry under autograd: the forward is the HIP path, the
    cotangents (dx, dA, dB, dscaling) are those of the reference's custom_vjp (quantized_lora.py:337-394),
    checked against the oracle's float32 pullback cast as the reference casts it."""
    import torch

    rng = np.random.default_rng(m + k)
    x = o.bf16_round(rng.standard_normal((m, k)).astype(F32))
    w = o.quantize_frozen_weight((rng.standard_normal((k, n)) * 0.05).astype(F32), bits=wb, group_size=group,
                                 scale_dtype="f32")
    a = o.bf16_round((rng.standard_normal((k, rank)) * 0.05).astype(F32))
    b = o.bf16_round((rng.standard_normal((rank, n)) * 0.05).astype(F32))
    dy = o.bf16_round(rng.standard_normal((m, n)).astype(F32))
    s = F32(1.25)
    want = o.quantized_lora_linear_bwd(x, w, a, b, s, dy)
    xt, at, bt = (_bf(dev, v).requires_grad_(True) for v in (x, a, b))
    st = torch.tensor(float(s), dtype=torch.float32, device=dev, requires_grad=True)
    out = pkg.quantized_lora.quantized_lora_linear(xt, _to_dev(pkg, dev, w), at, bt, st, activation_bits=ab)
    plain = pkg.quantized_lora.quantized_lora_linear(xt.detach(), _to_dev(pkg, dev, w), at.detach(), bt.detach(),
                                                     float(s), activation_bits=ab)
    assert torch.equal(out.detach().view(torch.int16), plain.view(torch.int16))
    out.backward(_bf(dev, dy))
    torch.cuda.synchronize()
    for name, got, ref in (("dx", xt.grad, want[0]), ("dA", at.grad, want[1]), ("dB", bt.grad, want[2])):
        rep = wc.compare(got.to(torch.float32).cpu().numpy(), ref)
        print(f"[gq backward parity] {name} {rep}", flush=True)
        assert rep["violations"] == 0, (name, rep)
    np.testing.assert_allclose(float(st.grad), float(want[3]), rtol=1e-3, atol=1e-3)
