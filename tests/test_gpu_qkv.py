"""GPU parity of the Qwen3.5 attention input stage (split, Q/K RMSNorm, partial RoPE behind the W8A8
QKV projection) against the oracle; bf16 outputs to |a - b| <= 2e-2 + 1e-2 |b|, copies bitwise."""

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


def _np(t):
    import torch

    torch.cuda.synchronize()
    return t.to(torch.float32).cpu().numpy()


@pytest.mark.parametrize("hq,hkv,d,rot,rows", [(4, 2, 4, 2, 6), (16, 4, 256, 64, 40), (8, 8, 128, 128, 33),
                                               (6, 2, 64, 0, 17), (2, 1, 130, 26, 9), (32, 8, 128, 64, 257)])
def test_split_norm_rope_matches_oracle(dev, pkg, hq, hkv, d, rot, rows):
    import torch

    w8 = pkg.w8a8_lora
    cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000.0, 1e-6)
    rng = np.random.default_rng(hq * 1000 + d)
    fused = o.bf16_round(rng.standard_normal((rows, cfg.fused_width)).astype(F32) * 2.0)
    qw, kw = (rng.standard_normal(d).astype(F32) * 0.1 for _ in range(2))
    pos = rng.integers(0, 40_000, rows).astype(np.int32)
    pos[0] = 0
    print(f"[case] qkv post hq={hq} hkv={hkv} d={d} rot={rot} rows={rows}", flush=True)
    got = w8.qkv_split_norm_rope(torch.from_numpy(fused).to(dev).to(torch.bfloat16), torch.from_numpy(qw).to(dev),
                                 torch.from_numpy(kw).to(dev), torch.from_numpy(pos).to(dev), cfg)
    want = o.qkv_split_norm_rope(fused, qw, kw, pos, num_query_heads=hq, num_kv_heads=hkv, head_dim=d,
                                 rotary_dim=rot, rope_theta=10_000.0, eps=1e-6)
    q, k, v, gate = (_np(t) for t in got)
    assert q.shape == (rows, hq, d) and k.shape == (rows, hkv, d) and v.shape == (rows, hkv, d)
    assert gate.shape == (rows, hq * d)
    np.testing.assert_array_equal(v, want[2])          # copies
    np.testing.assert_array_equal(gate, want[3])
    for name, u, t in (("q", q, want[0]), ("k", k, want[1])):
        rep = wc.compare(u, t)
        print(f"[parity] qkv {name} {rep}", flush=True)
        assert rep["violations"] == 0, (name, rep)
    # the pass-through part of a head and position 0 see no rotation: equal to the norm alone, bitwise
    if rot < d:
        np.testing.assert_array_equal(q[..., rot:], want[0][..., rot:])
    np.testing.assert_array_equal(q[0], want[0][0])


def test_full_stage_with_w8a8_projection(dev, pkg):
    """Decoder RMSNorm -> W8A8 QKV + two adapters -> split / norms / RoPE, batch x sequence shaped,
    in the geometry of the reference's own test (tests/tx/kernels/test_qwen3_5_qkv_lora.py:19-50)
    widened to K = 64, and at a Qwen3.5-like head geometry."""
    import torch

    w8, ql = pkg.w8a8_lora, pkg.quantized_lora
    for (hq, hkv, d, rot, k, batch, seq, rank) in [(4, 2, 4, 2, 64, 2, 3, 3), (8, 2, 128, 32, 512, 2, 24, 16)]:
        cfg = w8.Qwen35QKVStageConfig(hq, hkv, d, rot, 10_000.0, 1e-6)
        rng = np.random.default_rng(73 + d)
        hidden = o.bf16_round(rng.standard_normal((batch, seq, k)).astype(F32))
        inw, qw, kw = (rng.standard_normal(n).astype(F32) * 0.1 for n in (k, d, d))
        wq = o.quantize_frozen_weight(rng.standard_normal((k, cfg.fused_width)).astype(F32) * 0.2, bits=8,
                                      group_size=k, scale_dtype="f32")
        a = o.bf16_round(rng.standard_normal((2, k, rank)).astype(F32) * 0.2)
        b = o.bf16_round(rng.standard_normal((2, rank, cfg.fused_width)).astype(F32) * 0.2)
        s = np.asarray([0.75, 1.25], F32)
        idx = np.asarray([1, 0], np.int32)                      # one adapter per example
        pos = np.stack([np.arange(seq), np.arange(seq) + 7]).astype(np.int32)
        t = lambda v, dt=torch.bfloat16: torch.from_numpy(np.ascontiguousarray(v)).to(dev).to(dt)
        wt = ql.GroupQuantizedWeight(torch.from_numpy(wq.codes).to(dev), torch.from_numpy(wq.scales).to(dev), k, k, 8, k)
        with pytest.raises(RuntimeError, match="disabled by default"):
            w8.w8a8_qkv_lora_rope(t(hidden), t(inw, torch.float32), t(qw, torch.float32), t(kw, torch.float32), wt,
                                  t(a), t(b), t(s, torch.float32), t(pos, torch.int32), config=cfg)
        got = w8.w8a8_qkv_lora_rope(t(hidden), t(inw, torch.float32), t(qw, torch.float32), t(kw, torch.float32), wt,
                                    t(a), t(b), t(s, torch.float32), t(pos, torch.int32), config=cfg,
                                    adapter_indices=t(idx, torch.int32), enabled=True)
        want = o.w8a8_qkv_lora_rope(hidden.reshape(-1, k), inw, qw, kw, wq, a, b, s, np.repeat(idx, seq),
                                    pos.reshape(-1), num_query_heads=hq, num_kv_heads=hkv, head_dim=d,
                                    rotary_dim=rot, rope_theta=10_000.0, eps=1e-6)
        shapes = ((batch, seq, hq, d), (batch, seq, hkv, d), (batch, seq, hkv, d), (batch, seq, hq * d))
        for name, u, w_, shape in zip("qkvg", got, want, shapes):
            assert tuple(u.shape) == shape
            rep = wc.compare(_np(u).reshape(w_.shape), w_)
            assert rep["violations"] == 0, (name, rep)


def test_rejects_bad_geometry(dev, pkg):
    import torch

    w8 = pkg.w8a8_lora
    with pytest.raises(ValueError):
        w8.Qwen35QKVStageConfig(4, 3, 8, 4, 1e4, 1e-6)
    with pytest.raises(ValueError):
        w8.Qwen35QKVStageConfig(4, 2, 8, 3, 1e4, 1e-6)
    cfg = w8.Qwen35QKVStageConfig(4, 2, 8, 4, 1e4, 1e-6)
    fused = torch.zeros(3, cfg.fused_width, dtype=torch.bfloat16, device=dev)
    wgt = torch.zeros(8, device=dev)
    with pytest.raises(ValueError):
        w8.qkv_split_norm_rope(fused[:, :-8], wgt, wgt, torch.zeros(3, dtype=torch.int32, device=dev), cfg)
    with pytest.raises(ValueError):
        w8.qkv_split_norm_rope(fused, wgt, wgt, torch.zeros(4, dtype=torch.int32, device=dev), cfg)
    with pytest.raises(TypeError):
        w8.qkv_split_norm_rope(fused.float(), wgt, wgt, torch.zeros(3, dtype=torch.int32, device=dev), cfg)
    big = w8.Qwen35QKVStageConfig(2, 1, 1024, 4, 1e4, 1e-6)
    with pytest.raises(pkg._native.NativeError):
        w8.qkv_split_norm_rope(torch.zeros(1, big.fused_width, dtype=torch.bfloat16, device=dev),
                               torch.zeros(1024, device=dev), torch.zeros(1024, device=dev),
                               torch.zeros(1, dtype=torch.int32, device=dev), big)
