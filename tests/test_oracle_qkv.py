"""Pins for the oracle's Qwen3.5 attention input stage (skyrl/tx/kernels/qwen3_5_qkv_lora.py)."""

import numpy as np
import pytest

from oracle import w8a8_oracle as o

F32 = np.float32


def test_delta_rms_norm_against_torch():
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(0)
    x = o.bf16_round(rng.standard_normal((11, 48)).astype(F32))
    w = (rng.standard_normal(48) * 0.1).astype(F32)
    got = o.delta_rms_norm(x, w, 1e-6)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (48,), torch.from_numpy(1.0 + w.astype(np.float64)),
                                        1e-6).numpy()
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-3)) < 2 ** -8      # one bf16 rounding
    # zero delta, constant rows: x / |x| exactly
    ones = np.full((3, 16), 3.0, dtype=F32)
    np.testing.assert_allclose(o.delta_rms_norm(ones, np.zeros(16, F32), 1e-6), 1.0, rtol=4e-3)
    assert o.is_bf16_exact(got)


def test_partial_rope_is_a_complex_rotation():
    rng = np.random.default_rng(1)
    rows, heads, d, rot, theta = 5, 3, 16, 8, 10000.0
    x = o.bf16_round(rng.standard_normal((rows, heads, d)).astype(F32))
    pos = np.asarray([0, 1, 7, 100, 4095])
    got = o.apply_partial_rope(x, pos, rot, theta)
    half = rot // 2
    z = x[..., :half].astype(np.float64) + 1j * x[..., half:rot].astype(np.float64)
    ang = pos[:, None].astype(np.float64) / theta ** (2.0 * np.arange(half) / rot)
    zr = z * np.exp(1j * ang)[:, None, :]
    np.testing.assert_allclose(got[..., :half], zr.real, atol=2e-2, rtol=1e-2)
    np.testing.assert_allclose(got[..., half:rot], zr.imag, atol=2e-2, rtol=1e-2)
    np.testing.assert_array_equal(got[..., rot:], x[..., rot:])               # pass-through part
    np.testing.assert_array_equal(got[0], x[0])                               # position 0
    np.testing.assert_array_equal(o.apply_partial_rope(x, pos, 0, theta), x)  # no rotary dims
    # rotations preserve the norm of every (i, i + half) pair and compose additively
    n0 = np.hypot(x[..., :half], x[..., half:rot])
    n1 = np.hypot(got[..., :half], got[..., half:rot])
    np.testing.assert_allclose(n1, n0, atol=3e-2, rtol=1e-2)
    twice = o.apply_partial_rope(o.apply_partial_rope(x, pos, rot, theta), 2 * pos, rot, theta)
    once = o.apply_partial_rope(x, 3 * pos, rot, theta)
    np.testing.assert_allclose(twice, once, atol=6e-2, rtol=2e-2)
    sin, cos = o.rope_sin_cos(np.asarray([3]), 4, 100.0)
    np.testing.assert_allclose(sin[0], [np.sin(3.0), np.sin(0.3)], rtol=1e-6)
    np.testing.assert_allclose(cos[0], [np.cos(3.0), np.cos(0.3)], rtol=1e-6)


def test_interleaving_enumerated():
    """One kv head with two query heads, head_dim 2: columns are q0 g0 q1 g1 k v."""
    fused = np.arange(12, dtype=F32)[None, :] + 1.0
    q, k, v, gate = o.qkv_split_norm_rope(fused, np.zeros(2, F32), np.zeros(2, F32), np.asarray([0]),
                                          num_query_heads=2, num_kv_heads=1, head_dim=2, rotary_dim=0,
                                          rope_theta=10000.0, eps=1e-6)
    np.testing.assert_array_equal(gate, [[3, 4, 7, 8]])
    np.testing.assert_array_equal(v, [[[11, 12]]])
    norm = lambda a: o.bf16_round(np.asarray(a, F32) / np.sqrt(np.mean(np.square(a)) + 1e-6))
    np.testing.assert_allclose(q[0, 0], norm([1, 2]), rtol=4e-3)
    np.testing.assert_allclose(q[0, 1], norm([5, 6]), rtol=4e-3)
    np.testing.assert_allclose(k[0, 0], norm([9, 10]), rtol=4e-3)
    # two kv heads: the second group starts after the first group's v
    fused2 = np.arange(24, dtype=F32)[None, :]
    _, k2, v2, g2 = o.qkv_split_norm_rope(fused2, np.zeros(2, F32), np.zeros(2, F32), np.asarray([0]),
                                          num_query_heads=4, num_kv_heads=2, head_dim=2, rotary_dim=0,
                                          rope_theta=10000.0, eps=1e-6)
    np.testing.assert_array_equal(v2, [[[10, 11], [22, 23]]])
    np.testing.assert_array_equal(g2, [[2, 3, 6, 7, 14, 15, 18, 19]])


def test_w8a8_stage_is_the_composition():
    rng = np.random.default_rng(2)
    cfg = dict(num_query_heads=4, num_kv_heads=2, head_dim=8, rotary_dim=4, rope_theta=10000.0, eps=1e-6)
    width = 4 * 2 * 8 + 2 * 2 * 8
    k = 16
    hidden = o.bf16_round(rng.standard_normal((6, k)).astype(F32))
    w = o.quantize_frozen_weight(rng.standard_normal((k, width)).astype(F32), bits=8, group_size=k, scale_dtype="f32")
    a = o.bf16_round(rng.standard_normal((2, k, 3)).astype(F32) * 0.2)
    b = o.bf16_round(rng.standard_normal((2, 3, width)).astype(F32) * 0.2)
    s = np.asarray([0.75, 1.5], F32)
    idx = np.asarray([0, 1, 1, 0, 1, 0])
    pos = np.asarray([0, 1, 7, 3, 4, 9])
    inw, qw, kw = (rng.standard_normal(n).astype(F32) * 0.1 for n in (k, 8, 8))
    q, kk, v, gate = o.w8a8_qkv_lora_rope(hidden, inw, qw, kw, w, a, b, s, idx, pos, **cfg)
    assert q.shape == (6, 4, 8) and kk.shape == (6, 2, 8) and v.shape == (6, 2, 8) and gate.shape == (6, 32)
    fused = o.quantized_lora_linear_multi(o.delta_rms_norm(hidden, inw, 1e-6), w, a, b, s, idx)
    want = o.qkv_split_norm_rope(fused, qw, kw, pos, **cfg)
    for u, t in zip((q, kk, v, gate), want):
        np.testing.assert_array_equal(u, t)
    assert all(o.is_bf16_exact(t) for t in (q, kk, v, gate))
