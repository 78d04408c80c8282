"""Pins the CPU oracle against the reference's own golden vectors and against
what the mathematics fixes.  No GPU, no reference import."""

import hashlib
import itertools

import numpy as np
import pytest

from golden import host_case
from oracle import w8a8_oracle as o

F32 = np.float32


def _sha(b: bytes) -> str:
    return hashlib.sha256(b).hexdigest()


# -- the SHA-256 pinned host case (rocm/probe_w8a8_lora_forward.py:210-218) ------------

def test_host_case_inputs_match_reference_digests():
    c = host_case.build()
    pins = host_case.SPEC["sha256"]
    assert o.sha256_bf16(c["x"]) == pins["x"]
    assert _sha(c["weight_codes"].tobytes(order="C")) == pins["weight_codes"]
    assert o.sha256_bf16(c["weight_scales"]) == pins["weight_scales"]
    assert o.sha256_bf16(c["lora_a"]) == pins["lora_a"]
    assert o.sha256_bf16(c["lora_b"]) == pins["lora_b"]
    assert _sha(np.asarray(c["lora_scaling"], dtype=F32).tobytes()) == pins["lora_scaling"]


def test_host_case_expected_output_matches_reference_digest():
    c = host_case.build()
    out = o.quantized_lora_linear(c["x"], c["weight"], c["lora_a"], c["lora_b"], c["lora_scaling"])
    assert out.shape == (3, 32)
    expected = np.ascontiguousarray(out[:, : c["out_features"]])
    assert o.sha256_bf16(expected) == host_case.SPEC["sha256"]["expected"]
    # multi-adapter formulation with one adapter is the same function
    multi = o.quantized_lora_linear_multi(c["x"], c["weight"], c["lora_a"][None], c["lora_b"][None],
                                          np.asarray([c["lora_scaling"]]), np.zeros(3, np.int64))
    np.testing.assert_array_equal(o.bf16_bits(multi), o.bf16_bits(out))


def test_host_case_is_sensitive_to_every_operand():
    """Every input matters (> 3 % relative L2), as in probe_w8a8_lora_forward.py:1127-1190."""
    c = host_case.build()
    ref = o.quantized_lora_linear(c["x"], c["weight"], c["lora_a"], c["lora_b"], c["lora_scaling"])[:, :17]

    def rel(other):
        return np.linalg.norm(other[:, :17] - ref) / np.linalg.norm(ref)

    w = c["weight"]
    flipped = o.GroupQuantizedWeight(codes=(-w.codes).astype(np.int8), scales=w.scales,
                                     original_in_features=64, padded_in_features=64, bits=8, group_size=64)
    assert rel(o.quantized_lora_linear(c["x"], flipped, c["lora_a"], c["lora_b"], c["lora_scaling"])) > 0.03
    assert rel(o.quantized_lora_linear(c["x"], w, c["lora_a"], c["lora_b"], F32(0.0))) > 0.03
    assert rel(o.quantized_lora_linear(c["x"], w, c["lora_a"].T[::-1].T.copy(), c["lora_b"], c["lora_scaling"])) > 0.03
    assert rel(o.quantized_lora_linear(c["x"][::-1].copy(), w, c["lora_a"], c["lora_b"], c["lora_scaling"])) > 0.03
    scaled = o.GroupQuantizedWeight(codes=w.codes, scales=w.scales * F32(2), original_in_features=64,
                                    padded_in_features=64, bits=8, group_size=64)
    assert rel(o.quantized_lora_linear(c["x"], scaled, c["lora_a"], c["lora_b"], c["lora_scaling"])) > 0.03


# -- hand-coded vectors of tests/tx/kernels/test_quantized_lora.py:30-74 ----------------

def test_int4_pack_roundtrip_known_bytes():
    values = np.asarray([[-7, -1, 0], [-6, 1, 7], [-5, 2, 6], [-4, 3, 5]], dtype=np.int8)
    packed = o.pack_signed_int4(values)
    np.testing.assert_array_equal(packed, np.asarray([[0xA9, 0x1F, 0x70], [0xCB, 0x32, 0x56]], np.uint8))
    np.testing.assert_array_equal(o.unpack_signed_int4(packed), values)


def _w4():
    return o.GroupQuantizedWeight(codes=np.asarray([[0x31, 0x4E], [0x0B, 0x96]], np.uint8),
                                  scales=np.asarray([[0.5, 2.0], [1.5, 0.25]], F32),
                                  original_in_features=3, padded_in_features=4, bits=4, group_size=2)


def test_hand_coded_int4_dequant():
    expected = np.asarray([[0.5, -4.0], [1.5, 8.0], [-7.5, 1.5]], F32)
    np.testing.assert_array_equal(o.dequantize_frozen_weight(_w4()), expected)


def test_hand_coded_w4a4_grouped_linear():
    x = np.asarray([[7.0, -3.0, -7.0], [0.0, 0.0, 3.0]], F32)
    expected = np.asarray([[51.5, -62.5], [-22.5, 4.5]], F32)
    np.testing.assert_allclose(o.quantized_frozen_linear_f32(x, _w4(), activation_bits=4), expected,
                               rtol=1e-6, atol=1e-6)


# -- bf16 rounding against an independent implementation ---------------------------------

def test_bf16_round_matches_torch():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(1)
    a = np.concatenate([rng.standard_normal(4096).astype(F32) * F32(10) ** rng.integers(-20, 20, 4096).astype(F32),
                        np.asarray([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, np.inf, -np.inf], F32)])
    want = torch.from_numpy(a).to(torch.bfloat16).to(torch.float32).numpy()
    np.testing.assert_array_equal(o.bf16_round(a).view(np.uint32), want.view(np.uint32))
    # ties to even: 1 + 2^-8 is exactly between 1 and 1 + 2^-7
    assert o.bf16_round(F32(1.00390625)) == F32(1.0)
    assert o.bf16_round(F32(1.01171875)) == F32(1.015625)


# -- quantizer: closed forms, invariants, brute force -------------------------------------

def test_dynamic_quantizer_closed_forms():
    x = np.asarray([[127.0, -63.5, 0.5, 1.5, 2.5, -2.5, 0.0, 126.5]], F32)
    codes, scales = o.quantize_rows(x)
    assert scales[0] == F32(1.0)
    # rint is half-to-even: 0.5 -> 0, 1.5 -> 2, 2.5 -> 2, -2.5 -> -2, -63.5 -> -64, 126.5 -> 126
    np.testing.assert_array_equal(codes[0], np.asarray([127, -64, 0, 2, 2, -2, 0, 126], np.int8))
    z_codes, z_scales = o.quantize_rows(np.zeros((2, 8), F32))
    assert np.all(z_codes == 0) and np.all(z_scales == F32(1.0))


def test_dynamic_quantizer_brute_force_scalar():
    rng = np.random.default_rng(5)
    x = o.bf16_round(rng.standard_normal((7, 32)).astype(F32))
    codes, scales = o.quantize_rows(x)
    for m in range(7):
        amax = max(abs(float(v)) for v in x[m])
        s = F32(amax) / F32(127.0)
        assert scales[m] == s
        for k in range(32):
            q = np.rint(F32(x[m, k]) / s)
            assert codes[m, k] == int(max(-127, min(127, q)))
    assert np.all(np.abs(codes.astype(np.int32)).max(axis=1) == 127)


def test_int_matmul_brute_force_and_large_path():
    rng = np.random.default_rng(3)
    a = rng.integers(-127, 128, (5, 9), dtype=np.int8)
    b = rng.integers(-127, 128, (9, 4), dtype=np.int8)
    want = [[sum(int(a[i, k]) * int(b[k, j]) for k in range(9)) for j in range(4)] for i in range(5)]
    np.testing.assert_array_equal(o.int_matmul(a, b), np.asarray(want, np.int32))
    # extreme accumulators on the float64 path: all codes at +-127, K = 12288
    a2 = np.full((1400, 12288), 127, np.int8)
    b2 = np.full((12288, 2), -127, np.int8)
    b2[:, 1] = 127
    got = o.int_matmul(a2, b2)
    assert got.dtype == np.int32
    assert np.all(got[:, 0] == -12288 * 127 * 127) and np.all(got[:, 1] == 12288 * 127 * 127)
    a3 = rng.integers(-127, 128, (300, 300), dtype=np.int8)
    b3 = rng.integers(-127, 128, (300, 300), dtype=np.int8)
    np.testing.assert_array_equal(o.int_matmul(a3, b3), a3.astype(np.int32) @ b3.astype(np.int32))


def test_base_path_reduces_to_integer_matmul_with_unit_scales():
    rng = np.random.default_rng(4)
    # rows whose absmax is exactly 127 quantize to themselves with scale 1
    x = rng.integers(-127, 128, (6, 16)).astype(F32)
    x[:, 0] = 127.0
    wq = rng.integers(-127, 128, (16, 10), dtype=np.int8)
    w = o.GroupQuantizedWeight(codes=wq, scales=np.ones((1, 10), F32), original_in_features=16,
                               padded_in_features=16, bits=8, group_size=16)
    out, xc, xs, acc = o.quantized_frozen_linear_f32(x, w, return_parts=True)
    np.testing.assert_array_equal(xc[:, 0, :], x.astype(np.int8))
    np.testing.assert_array_equal(out, (x.astype(np.int32) @ wq.astype(np.int32)).astype(F32))


def test_zero_inputs_give_finite_zeros():
    w = o.quantize_frozen_weight(np.zeros((64, 8), F32), group_size=64)
    assert np.all(w.scales == 1.0) and np.all(w.codes == 0)
    out = o.quantized_lora_linear(np.zeros((3, 64), F32), w, np.zeros((64, 4), F32), np.zeros((4, 8), F32), 1.0)
    assert np.all(out == 0) and np.all(np.isfinite(out))


def test_single_cast_property():
    """out == bf16(base_f32 + s*low_f32) and differs from the early-cast variant somewhere
    (tests/tx/kernels/test_quantized_lora.py:178-199)."""
    rng = np.random.default_rng(11)
    x = o.bf16_round(rng.standard_normal((32, 128)).astype(F32))
    w = o.quantize_frozen_weight(rng.standard_normal((128, 48)).astype(F32), group_size=128, scale_dtype="f32")
    a = o.bf16_round(rng.standard_normal((128, 8)).astype(F32) * F32(0.1))
    b = o.bf16_round(rng.standard_normal((8, 48)).astype(F32) * F32(0.1))
    s = F32(1.25)
    out = o.quantized_lora_linear(x, w, a, b, s)
    base = o.quantized_frozen_linear_f32(x, w)
    low = (x @ a) @ b
    np.testing.assert_array_equal(out, o.bf16_round(base + low * s))
    early = o.bf16_round(o.bf16_round(base) + o.bf16_round(low * s))
    assert np.any(early != out)


def test_quantization_quality_bounds():
    """W8A8 relative L2 < 0.025 against the dense product and weight round trip < 0.012
    (tests/tx/kernels/test_quantized_lora.py:77-112), re-seeded."""
    rng = np.random.default_rng(8)
    wd = rng.standard_normal((70, 13)).astype(F32)
    w = o.quantize_frozen_weight(wd, bits=8, group_size=10, scale_dtype="f32")
    assert w.padded_in_features == 70
    rt = o.dequantize_frozen_weight(w)
    assert np.linalg.norm(rt - wd) / np.linalg.norm(wd) < 0.012
    x = rng.standard_normal((32, 64)).astype(F32)
    wd2 = rng.standard_normal((64, 24)).astype(F32)
    w2 = o.quantize_frozen_weight(wd2, bits=8, group_size=32, scale_dtype="f32")
    out = o.quantized_frozen_linear_f32(x, w2)
    dense = x @ wd2
    assert np.linalg.norm(out - dense) / np.linalg.norm(dense) < 0.025


def test_padded_k_and_multi_group_sum():
    rng = np.random.default_rng(9)
    wd = rng.standard_normal((5, 3)).astype(F32)
    w = o.quantize_frozen_weight(wd, bits=8, group_size=4, scale_dtype="f32")
    assert w.padded_in_features == 8 and w.codes.shape == (8, 3) and w.scales.shape == (2, 3)
    assert np.all(w.codes[5:] == 0)
    x = rng.standard_normal((2, 5)).astype(F32)
    out, xc, xs, acc = o.quantized_frozen_linear_f32(x, w, return_parts=True)
    manual = np.zeros((2, 3), F32)
    for g in range(2):
        manual += acc[:, g, :].astype(F32) * xs[:, g, None] * w.scales[g][None]
    np.testing.assert_array_equal(out, manual)


# -- multi-adapter LoRA closed forms (tests/tx/layers/test_lora_fast_path.py:21-49) -----

def _arange_lora(n=3, k=5, r=3, out=7):
    a = (np.arange(n * k * r, dtype=F32).reshape(n, k, r) / F32(97.0))
    b = (np.arange(n * r * out, dtype=F32).reshape(n, r, out) / F32(89.0))
    s = np.asarray([0.25, 0.75, 1.25], F32)
    return a, b, s


def test_lora_delta_single_adapter_matches_direct_formula():
    a, b, s = _arange_lora()
    x = np.arange(20, dtype=F32).reshape(4, 5) / F32(19.0)
    for adapter in (0, 2):
        got = o.lora_delta_multi(x, a, b, s, np.full(4, adapter))
        want = (x @ a[adapter]) @ b[adapter] * s[adapter]
        np.testing.assert_allclose(got, want, rtol=1e-6, atol=1e-6)


def test_lora_delta_multi_adapter_matches_per_row_brute_force():
    a, b, s = _arange_lora()
    x = np.arange(30, dtype=F32).reshape(6, 5) / F32(17.0)
    idx = np.asarray([2, 0, 1, 1, 2, 0])
    got = o.lora_delta_multi(x, a, b, s, idx)
    for m in range(6):
        want = np.zeros(7, np.float64)
        for n in range(7):
            for r in range(3):
                z = sum(float(x[m, k]) * float(a[idx[m], k, r]) for k in range(5))
                want[n] += z * float(b[idx[m], r, n])
        np.testing.assert_allclose(got[m], want * float(s[idx[m]]), rtol=1e-5)
    with pytest.raises(ValueError):
        o.lora_delta_multi(x, a, b, s, np.asarray([0, 1, 2, 3, 0, 0]))


def test_lora_equals_merged_weight_invariant():
    """out(x, adapter a) ~= x @ (W + s*A[a]@B[a]) (tests/tx/models/test_qwen3.py:123-180)."""
    rng = np.random.default_rng(42)
    x = rng.standard_normal((9, 16)).astype(F32)
    a = rng.standard_normal((2, 16, 4)).astype(F32)
    b = rng.standard_normal((2, 4, 6)).astype(F32)
    s = np.asarray([2.0, 2.0], F32)
    idx = rng.integers(0, 2, 9)
    delta = o.lora_delta_multi(x, a, b, s, idx)
    for m in range(9):
        merged = F32(2.0) * (a[idx[m]] @ b[idx[m]])
        np.testing.assert_allclose(delta[m], x[m] @ merged, rtol=1e-3, atol=1e-3)


# -- interleave, routing ---------------------------------------------------------------

def test_fuse_split_brute_force_and_roundtrip():
    q = np.arange(2 * 8).reshape(2, 8)          # groups of 4 (q_per_kv*hd = 4, 2 groups)
    k = 100 + np.arange(2 * 4).reshape(2, 4)    # groups of 2
    v = 200 + np.arange(2 * 4).reshape(2, 4)
    fused = o.fuse(q, k, v, group_sizes=(4, 2, 2))
    assert fused.shape == (2, 16)
    np.testing.assert_array_equal(fused[0], [0, 1, 2, 3, 100, 101, 200, 201, 4, 5, 6, 7, 102, 103, 202, 203])
    for got, want in zip(o.split(fused, (4, 2, 2)), (q, k, v)):
        np.testing.assert_array_equal(got, want)
    g = np.arange(6).reshape(1, 6)
    u = 10 + np.arange(6).reshape(1, 6)
    gu = o.fuse(g, u, group_sizes=(1, 1))
    np.testing.assert_array_equal(gu[0], [0, 10, 1, 11, 2, 12, 3, 13, 4, 14, 5, 15])
    np.testing.assert_array_equal(gu[:, 0::2], g)
    np.testing.assert_array_equal(gu[:, 1::2], u)


@pytest.mark.parametrize("group_sizes,group_offset,g_local,expected_scale", [
    ([2, 2, 2], 1, 2, [0, 0, 1, 1, 2, 2]),
    ([2, 2, 2], 0, 2, [1, 1, 2, 2, 0, 0]),
    ([2, 2, 2], 2, 1, [0, 0, 0, 0, 1, 1]),
    ([6], 0, 1, [1, 1, 1, 1, 1, 1]),
    ([2, 0, 0, 4], 1, 2, [0, 0, 0, 0, 0, 0]),
    ([1, 3, 2], 1, 2, [0, 1, 1, 1, 2, 2]),
])
def test_ragged_dot_group_offset_table(group_sizes, group_offset, g_local, expected_scale):
    """tests/tx/layers/test_ragged_dot.py:8-33."""
    lhs = np.arange(12, dtype=F32).reshape(6, 2)
    rhs = np.stack([(i + 1) * np.eye(2, dtype=F32) for i in range(g_local)])
    got = o.ragged_dot(lhs, rhs, np.asarray(group_sizes), group_offset=np.asarray([group_offset]))
    np.testing.assert_allclose(got, lhs * np.asarray(expected_scale, F32)[:, None])


def test_prepare_routing_is_a_stable_sort():
    idx = np.asarray([2, 0, 1, 0, 2, 1, 0])
    toks = np.arange(7)
    s, sizes, unsort, ad = o.prepare_routing(toks, idx, 4, adapter_indices=idx * 10)
    np.testing.assert_array_equal(s, [1, 3, 6, 2, 5, 0, 4])
    np.testing.assert_array_equal(sizes, [3, 2, 2, 0])
    np.testing.assert_array_equal(s[unsort], toks)
    np.testing.assert_array_equal(ad, [0, 0, 0, 10, 10, 20, 20])


# -- RMSNorm and SwiGLU closed forms ------------------------------------------------------

def test_rms_norm_closed_forms():
    # constant rows: mean(x^2) = c^2 exactly, x * rsqrt(c^2 + eps) rounds to +-1 in bf16
    x = np.full((2, 64), 3.0, F32)
    x[1] = -0.5
    np.testing.assert_array_equal(o.rms_norm(x, np.ones(64, F32)), np.sign(x))
    g = np.linspace(0.5, 1.5, 64).astype(F32)
    inv = F32(1) / np.sqrt(x[:, :1] ** 2 + F32(1e-6))
    np.testing.assert_array_equal(o.rms_norm(x, g), o.bf16_round((x * inv) * g))
    # one-hot row of length 4: mean = 1/4 -> rsqrt = 2 -> value 2
    one = np.zeros((1, 4), F32)
    one[0, 2] = 1.0
    np.testing.assert_array_equal(o.rms_norm(one, np.ones(4, F32), eps=0.0), [[0, 0, 2, 0]])
    # scale invariance up to bf16 rounding and eps
    rng = np.random.default_rng(2)
    y = o.bf16_round(rng.standard_normal((4, 256)).astype(F32))
    n1 = o.rms_norm(y, np.ones(256, F32))
    n2 = o.rms_norm(y * F32(4.0), np.ones(256, F32))
    assert np.max(np.abs(n1 - n2)) <= 2.0 ** -6
    rms = np.sqrt(np.mean(n1.astype(np.float64) ** 2, axis=1))
    np.testing.assert_allclose(rms, 1.0, atol=5e-3)


def test_silu_against_scipy_and_pairing_constant():
    special = pytest.importorskip("scipy.special")
    v = np.linspace(-30, 30, 2001).astype(F32)
    want = v.astype(np.float64) * special.expit(v.astype(np.float64))
    got = o.silu(v).astype(np.float64)
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) < 4e-7
    # pairing: gate = even column, up = odd column.  x = 1 (K = 64), W even = bf16(0.02),
    # odd = bf16(0.03): gate = 1.28125, up = 1.921875 -> bf16(silu(gate) * up) = 1.9296875;
    # the swapped pairing would give about 2.15.
    fused = np.tile(np.asarray([1.28125, 1.921875], F32), (3, 8))
    prod = o.swiglu_from_interleaved(fused)
    assert prod.shape == (3, 8)
    assert np.all(prod == F32(1.9296875))
    swapped = o.bf16_round(o.silu(F32(1.921875)) * F32(1.28125))
    assert abs(float(swapped.reshape(-1)[0]) - 2.15) < 0.01


def test_rms_gate_up_swiglu_pairing_end_to_end():
    """The closed form of tests/tx/kernels/rocm/test_bf16_rms_gate_up_lora_swiglu.py:335-364
    carried through the W8A8 composite: x = 1, gamma = 1, even columns 0.02, odd columns 0.03,
    A = B = 0.  Per-token quantization of an all-ones row is exact (code 127, scale 1/127);
    the weight codes are +-127 with scale w/127, so base = 64 * w up to f32 rounding."""
    k, pairs = 64, 8
    dense = np.zeros((k, 2 * pairs), F32)
    dense[:, 0::2] = o.bf16_round(F32(0.02))
    dense[:, 1::2] = o.bf16_round(F32(0.03))
    w = o.quantize_frozen_weight(dense, group_size=k, scale_dtype="f32")
    x = np.ones((4, k), F32)
    a = np.zeros((1, k, 8), F32)
    b = np.zeros((1, 8, 2 * pairs), F32)
    out, st = o.w8a8_rms_gate_up_lora_swiglu(x, np.ones(k, F32), w, a, b, np.ones(1, F32),
                                            np.zeros(4, np.int64), return_stages=True)
    assert np.all(st["normalized"] == 1.0)
    assert np.all(st["fused"][:, 0::2] == F32(1.28125)) and np.all(st["fused"][:, 1::2] == F32(1.921875))
    assert np.all(out == F32(1.9296875))


# -- MoE routing --------------------------------------------------------------------------

def test_moe_route_against_torch_topk_and_scipy_softmax():
    torch = pytest.importorskip("torch")
    special = pytest.importorskip("scipy.special")
    rng = np.random.default_rng(6)
    logits = rng.standard_normal((64, 16)).astype(F32)
    wts, sel = o.moe_route(logits, 4)
    probs = special.softmax(logits.astype(np.float64), axis=-1)
    tv, ti = torch.topk(torch.from_numpy(probs), 4, dim=-1)
    np.testing.assert_array_equal(sel, ti.numpy())
    want = tv.numpy() / tv.numpy().sum(-1, keepdims=True)
    np.testing.assert_allclose(wts, want, rtol=2e-6)
    np.testing.assert_allclose(wts.sum(-1), 1.0, rtol=1e-6)


def test_moe_expert_mlp_matches_per_token_brute_force():
    rng = np.random.default_rng(7)
    t, h, inter, e, topk, r = 12, 32, 16, 4, 2, 4
    hidden = o.bf16_round(rng.standard_normal((t, h)).astype(F32))
    logits = rng.standard_normal((t, e)).astype(F32)
    gu = [o.GroupQuantizedWeight(rng.integers(-127, 128, (h, 2 * inter), dtype=np.int8),
                                 rng.uniform(0.001, 0.01, (1, 2 * inter)).astype(F32), h, h, 8, h) for _ in range(e)]
    dn = [o.GroupQuantizedWeight(rng.integers(-127, 128, (inter, h), dtype=np.int8),
                                 rng.uniform(0.001, 0.01, (1, h)).astype(F32), inter, inter, 8, inter) for _ in range(e)]
    gua = o.bf16_round(rng.standard_normal((e, h, r)).astype(F32) * F32(0.02))
    gub = o.bf16_round(rng.standard_normal((e, r, 2 * inter)).astype(F32) * F32(0.02))
    da = o.bf16_round(rng.standard_normal((e, inter, r)).astype(F32) * F32(0.02))
    db = o.bf16_round(rng.standard_normal((e, r, h)).astype(F32) * F32(0.02))
    out = o.moe_expert_mlp(hidden, logits, topk, gu, dn, gua, gub, da, db, F32(1.0))
    wts, sel = o.moe_route(logits, topk)
    want = np.zeros((t, h), F32)
    for tok in range(t):
        acc = np.zeros(h, F32)
        for j in range(topk):
            ex = int(sel[tok, j])
            fused = o.quantized_lora_linear(hidden[tok:tok + 1], gu[ex], gua[ex], gub[ex], F32(1.0))
            act = o.swiglu_from_interleaved(fused)
            down = o.quantized_lora_linear(act, dn[ex], da[ex], db[ex], F32(1.0))
            acc = acc + down[0] * wts[tok, j]
        want[tok] = acc
    np.testing.assert_allclose(out, o.bf16_round(want), rtol=1e-2, atol=1e-5)


def test_numerical_gate_thresholds():
    e = np.linspace(-4, 4, 101)
    assert o.numerical_gate(e, e)["passed"]
    assert not o.numerical_gate(e + 0.3, e)["passed"]       # max-abs
    assert not o.numerical_gate(e * 1.02, e)["passed"]      # relative L2
    bad = e.copy()
    bad[0] = np.nan
    assert not o.numerical_gate(bad, e)["passed"]
    assert o.within_tolerance(np.asarray([1.0299]), np.asarray([1.0]))[0]
    assert not o.within_tolerance(np.asarray([1.031]), np.asarray([1.0]))[0]
