"""NumPy restatement of the reference's W8A8 LoRA linear forward semantics.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Every function cites the
reference file:line (relative to the reference checkout) whose arithmetic it
follows.  bf16 values are carried as float32 arrays whose low 16 mantissa bits
are zero; ``bf16_round`` is the only place a bf16 rounding happens.

How each function is pinned (the tests that do it live in ``tests/test_oracle_*.py``):

* ``bf16_round``/``bf16_bits``, ``quantize_frozen_weight``, ``dynamic_group_quantize``,
  ``quantized_frozen_linear_f32``, ``quantized_lora_linear``: the reference's
  SHA-256-pinned deterministic host case (rocm/probe_w8a8_lora_forward.py:210-218)
  plus the hand-coded int4 / W4A4 vectors of tests/tx/kernels/test_quantized_lora.py:30-74.
* ``int_matmul``: brute force in Python integers and the int32 ``numpy.matmul``.
* ``lora_delta_multi``/``quantized_lora_linear_multi``: the arange closed forms of
  tests/tx/layers/test_lora_fast_path.py:21-49 and per-row brute force.
* ``fuse``/``split``: brute force and round trip (skyrl/tx/layers/lora.py:325-351).
* ``ragged_dot``: the six-row table of tests/tx/layers/test_ragged_dot.py:8-33.
* ``swiglu_from_interleaved``: the pairing constant 1.9296875 derived from
  tests/tx/kernels/rocm/test_bf16_rms_gate_up_lora_swiglu.py:335-364.
* ``rms_norm``: closed forms (constant rows, power-of-two rows).  PARITY UNPINNED
  in the last f32 bit against XLA-CPU: the reference's ``jnp.mean`` reduction order
  and ``lax.rsqrt`` rounding live in jaxlib, which is not available; this oracle
  fixes mean = f32(sum_f64(x*x)/K) and rsqrt = 1/sqrt with IEEE f32 ops.
* ``silu``: exp/logistic rounding of XLA-CPU is likewise unavailable; PARITY
  UNPINNED in the last f32 bit, pinned to 1 ulp by the closed-form constant above
  and by ``scipy.special.expit``.
* ``quantized_lora_linear_bwd*``: ``torch.autograd`` (float64, CPU) through the straight-through
  function ``x @ dequant(W) + s * (x @ A) @ B``, central finite differences of the LoRA
  terms, and the zero/linearity identities of the equations.  PARITY UNPINNED in the float32
  summation order of XLA (float64 accumulation here).
* ``swiglu_pullback_interleaved``/``rms_norm_pullback``/``w8a8_rms_gate_up_lora_swiglu_bwd``:
  ``torch.autograd`` (float64, CPU) through ``silu(g) * u`` and through the smooth RMSNorm, the
  closed forms at g = 0 (d_gate = c u / 2, d_up = 0) and for a constant row (dx = 0 when dn * gamma
  is parallel to x), and the orthogonality sum(x * dx) ~ eps-term; the composite against autograd
  through the whole smooth function on bf16-exact inputs.  exp, the float32 reduction order and
  rsqrt of XLA are not available: PARITY UNPINNED in their last float32 bits.
* ``delta_rms_norm``/``apply_partial_rope``/``qkv_split_norm_rope``: ``torch.nn.functional.rms_norm``,
  the rotation written as a complex product, its group law R(p)R(q) = R(p + q), norm
  preservation, position 0 and ``rotary_dim`` 0 identities, and an enumerated interleaving
  (tests/tx/kernels/test_qwen3_5_qkv_lora.py:75-83 states it as ``FusedLoRALinear.split``).
  sin/cos/pow of XLA-CPU are not available: PARITY UNPINNED in their last float32 bits.
* ``apply_partial_rope_transpose``/``delta_rms_norm_vjp``/``qkv_split_norm_rope_bwd``/
  ``w8a8_qkv_lora_rope_bwd``: the adjoint identity <R x, y> = <x, R^T y> and R^T R = 1 of the rotation,
  ``torch.autograd`` (float64, CPU) through the smooth RMSNorm with ``1 + weight`` for dx and dweight,
  the re-interleave as the exact adjoint of the split (enumerated), and the composite against
  autograd through the whole smooth stage on bf16-exact inputs.  PARITY UNPINNED in the last
  float32 bits of XLA's reductions, rsqrt, sin, cos and pow.
* ``moe_combine_bwd``/``moe_route_bwd``/``moe_expert_mlp_bwd``: ``torch.autograd`` (float64, CPU) through
  the gather-weighted sum, through softmax / gather / renormalise with the selection held fixed, and
  through the whole smooth expert MLP on bf16-exact inputs; zero and linearity identities.
* ``moe_route``/``moe_combine``/``moe_expert_mlp``: ``torch.topk``/``scipy.special.softmax`` special
  cases and the merged-weight invariant of tests/tx/models/test_qwen3.py:123-180.
"""

from __future__ import annotations

import hashlib
from dataclasses import dataclass

import numpy as np

F32 = np.float32


# ---------------------------------------------------------------------------
# bf16 helpers
# ---------------------------------------------------------------------------
# Qwen3.5 attention input stage after the fused projection
# (skyrl/tx/kernels/qwen3_5_qkv_lora.py:88-95, 119-145, 216-286)
# ---------------------------------------------------------------------------

def delta_rms_norm(x, weight, eps: float) -> np.ndarray:
    """qwen3_5_qkv_lora.py:88-95: float32 statistics, multiplier ``1 + weight``, cast to bf16.
    mean and rsqrt are fixed as in ``rms_norm`` (PARITY UNPINNED in the last float32 bit)."""
    return rms_norm(x, (F32(1.0) + np.asarray(weight, dtype=F32)).astype(F32), eps)


def rope_sin_cos(positions, rotary_dim: int, rope_theta: float):
    """qwen3_5_qkv_lora.py:119-127: angle[p, i] = p / theta ** (2 i / rotary_dim), float32."""
    fraction = (F32(2.0) * np.arange(0, rotary_dim // 2, dtype=F32) / F32(rotary_dim)).astype(F32)
    timescale = np.power(F32(rope_theta), fraction).astype(F32)
    angles = (np.asarray(positions).astype(F32)[..., None] / timescale).astype(F32)
    return np.sin(angles).astype(F32), np.cos(angles).astype(F32)


def apply_partial_rope(x, positions, rotary_dim: int, rope_theta: float) -> np.ndarray:
    """qwen3_5_qkv_lora.py:130-145.  ``x`` is [..., heads, head_dim] (bf16 values), ``positions``
    [...]: the first ``rotary_dim`` entries of a head are rotated in halves (i, i + rotary_dim / 2),
    the products are float32, the result is cast to bf16 once; the rest passes through."""
    x = np.asarray(x, dtype=F32)
    if rotary_dim == 0:
        return x.copy()
    half = rotary_dim // 2
    first, second = x[..., :half], x[..., half:rotary_dim]
    sin, cos = rope_sin_cos(positions, rotary_dim, rope_theta)
    sin, cos = sin[..., None, :], cos[..., None, :]
    out = x.copy()
    out[..., :half] = bf16_round((first * cos).astype(F32) - (second * sin).astype(F32))
    out[..., half:rotary_dim] = bf16_round((first * sin).astype(F32) + (second * cos).astype(F32))
    return out


def qkv_split_norm_rope(fused, q_norm_weight, k_norm_weight, positions, *, num_query_heads: int,
                        num_kv_heads: int, head_dim: int, rotary_dim: int, rope_theta: float, eps: float):
    """qwen3_5_qkv_lora.py:266-286 on an interleaved fused projection [rows, width] (bf16 values):
    per kv head one group of ``queries_per_kv`` (q, gate) chunk pairs, then k, then v.  Returns
    q [rows, Hq, D], k [rows, Hkv, D], v [rows, Hkv, D], gate [rows, Hq * D]."""
    fused = np.asarray(fused, dtype=F32)
    rows = fused.shape[0]
    qpk = num_query_heads // num_kv_heads
    q_raw, k_raw, v_raw = split(fused, (qpk * 2 * head_dim, head_dim, head_dim))
    q_and_gate = q_raw.reshape(rows, num_query_heads, 2 * head_dim)
    q_raw, gate = q_and_gate[..., :head_dim], q_and_gate[..., head_dim:]
    k_raw = k_raw.reshape(rows, num_kv_heads, head_dim)
    v = v_raw.reshape(rows, num_kv_heads, head_dim)
    q = delta_rms_norm(q_raw.reshape(-1, head_dim), q_norm_weight, eps).reshape(q_raw.shape)
    k = delta_rms_norm(k_raw.reshape(-1, head_dim), k_norm_weight, eps).reshape(k_raw.shape)
    q = apply_partial_rope(q, positions, rotary_dim, rope_theta)
    k = apply_partial_rope(k, positions, rotary_dim, rope_theta)
    return q, k, v.copy(), gate.reshape(rows, num_query_heads * head_dim).copy()


def w8a8_qkv_lora_rope(hidden, input_norm_weight, q_norm_weight, k_norm_weight, weight: GroupQuantizedWeight,
                       lora_a, lora_b, lora_scaling, adapter_indices, positions, **config):
    """The stage with the W8A8 projection in the place of the bf16 one: delta RMSNorm -> W8A8 +
    LoRA (one cast) -> split, Q/K norms, partial RoPE.  ``hidden`` is [rows, K]."""
    eps = config["eps"]
    normalized = delta_rms_norm(hidden, input_norm_weight, eps)
    if lora_a is None:
        fused = quantized_frozen_linear(normalized, weight)
    else:
        fused = quantized_lora_linear_multi(normalized, weight, lora_a, lora_b, lora_scaling, adapter_indices)
    return qkv_split_norm_rope(fused, q_norm_weight, k_norm_weight, positions, **config)


# ---------------------------------------------------------------------------
# pull-back of the Qwen3.5 attention input stage (qwen3_5_qkv_lora.py:97-116, 148-164, 360-451)
# ---------------------------------------------------------------------------

def apply_partial_rope_transpose(dy, positions, rotary_dim: int, rope_theta: float) -> np.ndarray:
    """qwen3_5_qkv_lora.py:148-164: the transposed rotation on a bf16 cotangent [..., heads, head_dim]:
    [first cos + second sin, -first sin + second cos] in float32, one cast; the rest passes through."""
    dy = np.asarray(dy, dtype=F32)
    if rotary_dim == 0:
        return dy.copy()
    half = rotary_dim // 2
    first, second = dy[..., :half], dy[..., half:rotary_dim]
    sin, cos = rope_sin_cos(positions, rotary_dim, rope_theta)
    sin, cos = sin[..., None, :], cos[..., None, :]
    out = dy.copy()
    out[..., :half] = bf16_round((first * cos).astype(F32) + (second * sin).astype(F32))
    out[..., half:rotary_dim] = bf16_round((-first * sin).astype(F32) + (second * cos).astype(F32))
    return out


def delta_rms_norm_vjp(x, weight, dy, eps: float):
    """qwen3_5_qkv_lora.py:97-116 on rows [rows, width] (bf16 values): float32 statistics with the
    forward's mean and rsqrt rule, dx = bf16(inv * (dy (1 + w) - n * mean(dy (1 + w) n))) and the
    float32 weight cotangent sum_rows(dy * n) (summed in float64, rounded once; the reference's
    float32 reduction order is XLA's: PARITY UNPINNED in its last bits)."""
    x = np.asarray(x, dtype=F32)
    dy = np.asarray(dy, dtype=F32)
    ew = (F32(1.0) + np.asarray(weight, dtype=F32)).astype(F32)
    width = x.shape[-1]
    ssq = np.sum(x.astype(np.float64) * x.astype(np.float64), axis=-1, keepdims=True)
    inv = (F32(1.0) / np.sqrt(((ssq / np.float64(width)).astype(F32) + F32(eps)).astype(F32))).astype(F32)
    normalized = (x * inv).astype(F32)
    weighted = (dy * ew).astype(F32)
    prod = (weighted * normalized).astype(F32)
    mu = (np.sum(prod.astype(np.float64), axis=-1, keepdims=True) / np.float64(width)).astype(F32)
    dx = (inv * (weighted - (normalized * mu).astype(F32)).astype(F32)).astype(F32)
    dweight = np.sum((dy * normalized).astype(F32).astype(np.float64).reshape(-1, width), axis=0).astype(F32)
    return bf16_round(dx), dweight


def qkv_split_norm_rope_bwd(fused, q_norm_weight, k_norm_weight, positions, dq, dk, dv, dgate, *,
                            num_query_heads: int, num_kv_heads: int, head_dim: int, rotary_dim: int,
                            rope_theta: float, eps: float):
    """qwen3_5_qkv_lora.py:389-425: from the raw projection [rows, width] and the four output
    cotangents to the cotangent of the projection (bf16 values) and the float32 cotangents of the
    two head-norm weights."""
    fused = np.asarray(fused, dtype=F32)
    rows = fused.shape[0]
    qpk = num_query_heads // num_kv_heads
    q_proj, k_proj, _ = split(fused, (qpk * 2 * head_dim, head_dim, head_dim))
    q_raw = q_proj.reshape(rows, num_query_heads, 2 * head_dim)[..., :head_dim]
    k_raw = k_proj.reshape(rows, num_kv_heads, head_dim)
    dq = apply_partial_rope_transpose(np.asarray(dq, dtype=F32).reshape(rows, num_query_heads, head_dim),
                                      positions, rotary_dim, rope_theta)
    dk = apply_partial_rope_transpose(np.asarray(dk, dtype=F32).reshape(rows, num_kv_heads, head_dim),
                                      positions, rotary_dim, rope_theta)
    dq_raw, dq_w = delta_rms_norm_vjp(q_raw.reshape(-1, head_dim), q_norm_weight, dq.reshape(-1, head_dim), eps)
    dk_raw, dk_w = delta_rms_norm_vjp(k_raw.reshape(-1, head_dim), k_norm_weight, dk.reshape(-1, head_dim), eps)
    dq_proj = np.concatenate([dq_raw.reshape(rows, num_query_heads, head_dim),
                              np.asarray(dgate, dtype=F32).reshape(rows, num_query_heads, head_dim)],
                             axis=-1).reshape(rows, num_query_heads * 2 * head_dim)
    dfused = fuse(dq_proj, dk_raw.reshape(rows, num_kv_heads * head_dim),
                  np.asarray(dv, dtype=F32).reshape(rows, num_kv_heads * head_dim),
                  group_sizes=(qpk * 2 * head_dim, head_dim, head_dim))
    return dfused, dq_w, dk_w


def w8a8_qkv_lora_rope_bwd(hidden, input_norm_weight, q_norm_weight, k_norm_weight, weight: GroupQuantizedWeight,
                           lora_a, lora_b, lora_scaling, adapter_indices, positions, dq, dk, dv, dgate,
                           relaxed_weight: bool = True, **config):
    """The structure of _qwen35_qkv_lora_rope_bwd (qwen3_5_qkv_lora.py:360-451) with the quantized
    projection's own rule in the middle (``quantized_lora_linear_multi_bwd``).  Returns a dict with
    dhidden, d_input_norm_weight, d_q_norm_weight, d_k_norm_weight, d_lora_a, d_lora_b, d_lora_scaling
    and the intermediate dfused."""
    eps = config["eps"]
    normalized = delta_rms_norm(hidden, input_norm_weight, eps)
    if lora_a is None:
        fused = quantized_frozen_linear(normalized, weight)
    else:
        fused = quantized_lora_linear_multi(normalized, weight, lora_a, lora_b, lora_scaling, adapter_indices)
    dfused, dq_w, dk_w = qkv_split_norm_rope_bwd(fused, q_norm_weight, k_norm_weight, positions, dq, dk, dv, dgate,
                                                 **config)
    if lora_a is None:
        dn = bf16_round(_mm64(dfused, pullback_weight(weight, relaxed_weight).T))
        da = db = ds = None
    else:
        dn, da, db, ds = quantized_lora_linear_multi_bwd(normalized, weight, lora_a, lora_b, lora_scaling,
                                                         adapter_indices, dfused, relaxed_weight)
    dhidden, d_in_w = delta_rms_norm_vjp(hidden, input_norm_weight, dn, eps)
    return {"dhidden": dhidden, "d_input_norm_weight": d_in_w, "d_q_norm_weight": dq_w, "d_k_norm_weight": dk_w,
            "d_lora_a": da, "d_lora_b": db, "d_lora_scaling": ds, "dfused": dfused, "fused": fused,
            "normalized": normalized, "d_normalized": dn}


# ---------------------------------------------------------------------------

def bf16_bits(a) -> np.ndarray:
    """float32 -> uint16 bf16 bit pattern, round-to-nearest-even (NaN kept quiet)."""
    a = np.ascontiguousarray(np.asarray(a, dtype=F32))
    u = a.view(np.uint32)
    rounded = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)
    nan = np.isnan(a)
    if np.any(nan):
        rounded = np.where(nan, (u >> np.uint32(16)) | np.uint32(0x40), rounded)
    return rounded.astype(np.uint16)


def bf16_from_bits(bits) -> np.ndarray:
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(F32)


def bf16_round(a) -> np.ndarray:
    """Round float32 values to the nearest bf16 (ties to even), returned as float32."""
    return bf16_from_bits(bf16_bits(a))


def is_bf16_exact(a) -> bool:
    a = np.ascontiguousarray(np.asarray(a, dtype=F32))
    return bool(np.all((a.view(np.uint32) & np.uint32(0xFFFF)) == 0))


def sha256_bf16(a) -> str:
    return hashlib.sha256(bf16_bits(a).tobytes(order="C")).hexdigest()


# ---------------------------------------------------------------------------
# storage format (skyrl/tx/kernels/quantized_lora.py:20-91)
# ---------------------------------------------------------------------------

@dataclass(frozen=True)
class GroupQuantizedWeight:
    """K x N weight grouped along K; skyrl/tx/kernels/quantized_lora.py:20-41."""

    codes: np.ndarray
    scales: np.ndarray
    original_in_features: int
    padded_in_features: int
    bits: int
    group_size: int


def _validate_bits(bits: int) -> None:
    if bits not in (4, 8):
        raise ValueError(f"bits must be 4 or 8, got {bits}")


def _validate_group_size(group_size: int) -> None:
    if group_size <= 0 or group_size % 2:
        raise ValueError(f"group_size must be a positive even integer, got {group_size}")


def validate_quantized_weight(weight: GroupQuantizedWeight) -> None:
    """skyrl/tx/kernels/quantized_lora.py:56-91."""
    _validate_bits(weight.bits)
    _validate_group_size(weight.group_size)
    if weight.original_in_features <= 0 or weight.padded_in_features <= 0:
        raise ValueError("quantized weight input dimensions must be positive")
    if weight.padded_in_features < weight.original_in_features:
        raise ValueError("padded_in_features must be at least original_in_features")
    if weight.padded_in_features % weight.group_size:
        raise ValueError("padded_in_features must be divisible by group_size")
    if weight.codes.ndim != 2 or weight.scales.ndim != 2:
        raise ValueError("quantized weight codes and scales must both be rank-two")
    rows = weight.padded_in_features // (2 if weight.bits == 4 else 1)
    scale_shape = (weight.padded_in_features // weight.group_size, weight.codes.shape[1])
    if weight.codes.shape[0] != rows:
        raise ValueError(f"code rows {weight.codes.shape[0]} do not match expected {rows}")
    if weight.scales.shape != scale_shape:
        raise ValueError(f"scale shape {weight.scales.shape} does not match expected {scale_shape}")
    if weight.codes.shape[1] <= 0:
        raise ValueError("quantized weight output dimension must be positive")
    want = np.uint8 if weight.bits == 4 else np.int8
    if weight.codes.dtype != want:
        raise TypeError(f"W{weight.bits} codes must have dtype {want}, got {weight.codes.dtype}")
    if not np.issubdtype(weight.scales.dtype, np.floating):
        raise TypeError(f"quantized weight scales must be floating point, got {weight.scales.dtype}")


def pack_signed_int4(values) -> np.ndarray:
    """skyrl/tx/kernels/quantized_lora.py:94-109 (low nibble = even row, high = odd row)."""
    values = np.asarray(values)
    if values.ndim < 1 or values.shape[0] == 0 or values.shape[0] % 2:
        raise ValueError("signed INT4 packing requires an even, nonempty axis zero")
    if not np.issubdtype(values.dtype, np.integer):
        raise TypeError(f"signed INT4 values must be integral, got {values.dtype}")
    low = (values[0::2].astype(np.int16) & 0xF).astype(np.uint8)
    high = (values[1::2].astype(np.int16) & 0xF).astype(np.uint8)
    return low | (high << np.uint8(4))


def unpack_signed_int4(packed) -> np.ndarray:
    """skyrl/tx/kernels/quantized_lora.py:112-125."""
    packed = np.asarray(packed)
    if packed.ndim < 1 or packed.shape[0] == 0:
        raise ValueError("signed INT4 input must have a nonempty axis zero")
    if packed.dtype != np.uint8:
        raise TypeError(f"packed signed INT4 values must be uint8, got {packed.dtype}")
    low = (packed & np.uint8(0xF)).astype(np.int16)
    high = (packed >> np.uint8(4)).astype(np.int16)
    low = np.where(low >= 8, low - 16, low).astype(np.int8)
    high = np.where(high >= 8, high - 16, high).astype(np.int8)
    inter = np.stack((low, high), axis=1)
    return inter.reshape((packed.shape[0] * 2, *packed.shape[1:]))


def quantize_frozen_weight(weight, *, bits: int = 8, group_size: int = 64,
                           scale_dtype: str = "bf16") -> GroupQuantizedWeight:
    """Symmetric per-(group, output) weight quantizer; quantized_lora.py:128-171.

    ``scale_dtype`` is "bf16" (the reference default: scales are *stored* rounded
    to bf16 while the codes were computed with the f32 scale) or "f32".
    """
    _validate_bits(bits)
    _validate_group_size(group_size)
    weight = np.asarray(weight)
    if weight.ndim != 2:
        raise ValueError(f"weight must have shape [K, N], got {weight.shape}")
    if weight.shape[0] <= 0 or weight.shape[1] <= 0:
        raise ValueError(f"weight dimensions must be positive, got {weight.shape}")
    if not np.issubdtype(weight.dtype, np.floating):
        raise TypeError(f"weight must be floating point, got {weight.dtype}")
    if scale_dtype not in ("bf16", "f32"):
        raise TypeError(f"scale_dtype must be 'bf16' or 'f32', got {scale_dtype}")
    k, n = weight.shape
    k_pad = ((k + group_size - 1) // group_size) * group_size
    padded = np.zeros((k_pad, n), dtype=F32)
    padded[:k] = weight.astype(F32)
    grouped = padded.reshape((-1, group_size, n))
    qmax = (1 << (bits - 1)) - 1
    amax = np.max(np.abs(grouped), axis=1)
    with np.errstate(divide="ignore", invalid="ignore"):
        scales = np.where(amax > 0, amax / F32(qmax), F32(1.0)).astype(F32)
        q = np.clip(np.rint(grouped / scales[:, None, :]), -qmax, qmax).astype(np.int8)
    q = q.reshape((k_pad, n))
    codes = q if bits == 8 else pack_signed_int4(q)
    stored = bf16_round(scales) if scale_dtype == "bf16" else scales
    return GroupQuantizedWeight(codes=codes, scales=stored, original_in_features=k,
                                padded_in_features=k_pad, bits=bits, group_size=group_size)


def unpacked_codes(weight: GroupQuantizedWeight) -> np.ndarray:
    """quantized_lora.py:174-177."""
    validate_quantized_weight(weight)
    codes = weight.codes if weight.bits == 8 else unpack_signed_int4(weight.codes)
    return codes[: weight.padded_in_features].astype(np.int8)


def dequantize_frozen_weight(weight: GroupQuantizedWeight) -> np.ndarray:
    """quantized_lora.py:180-196 (float32 result)."""
    codes = unpacked_codes(weight)
    n = codes.shape[1]
    grouped = codes.reshape((-1, weight.group_size, n)).astype(F32)
    deq = grouped * weight.scales.astype(F32)[:, None, :]
    return deq.reshape((weight.padded_in_features, n))[: weight.original_in_features]


# ---------------------------------------------------------------------------
# activation quantizer and integer GEMM
# ---------------------------------------------------------------------------

def dynamic_group_quantize(x, bits: int = 8, group_size: int | None = None):
    """Per-(row, group) symmetric dynamic quantizer; quantized_lora.py:199-212.

    Both divisions are IEEE float32 divisions and ``rint`` rounds half to even.
    Returns (codes int8 [M, G, group_size], scales float32 [M, G]).
    """
    x = np.asarray(x, dtype=F32)
    if group_size is None:
        group_size = x.shape[1]
    qmax = (1 << (bits - 1)) - 1
    grouped = x.reshape((x.shape[0], x.shape[1] // group_size, group_size))
    amax = np.max(np.abs(grouped), axis=-1)
    scales = np.where(amax > 0, amax / F32(qmax), F32(1.0)).astype(F32)
    codes = np.clip(np.rint(grouped / scales[..., None]), -qmax, qmax).astype(np.int8)
    return codes, scales


def quantize_rows(x):
    """Per-token (group = whole row) A8 quantizer: (codes int8 [M,K], scales f32 [M])."""
    codes, scales = dynamic_group_quantize(x, 8, None)
    return codes[:, 0, :], scales[:, 0]


def int_matmul(a_codes, b_codes) -> np.ndarray:
    """Exact int8 x int8 -> int32 matrix product (quantized_lora.py:240-245).

    Small problems use numpy's int32 matmul.  Large ones go through float64 BLAS,
    which is exact here: |sum| <= K * 127^2 < 2^53 for any K below 5.5e11.
    """
    a = np.asarray(a_codes)
    b = np.asarray(b_codes)
    if a.shape[0] * a.shape[1] * b.shape[1] <= (1 << 24):
        return np.matmul(a.astype(np.int32), b.astype(np.int32), dtype=np.int32)
    out = np.empty((a.shape[0], b.shape[1]), dtype=np.int32)
    b64 = b.astype(np.float64)
    step = max(1, (1 << 27) // max(1, a.shape[1]))
    for r0 in range(0, a.shape[0], step):
        out[r0:r0 + step] = np.rint(a[r0:r0 + step].astype(np.float64) @ b64).astype(np.int32)
    return out


def quantized_frozen_linear_f32(x, weight: GroupQuantizedWeight, *, activation_bits: int = 8,
                                return_parts: bool = False):
    """FP32 epilogue input of the grouped quantized linear; quantized_lora.py:215-254.

    ``scaled = f32(acc) * x_scale * w_scale`` is evaluated left to right and the
    groups are summed in float32 in group order.
    """
    _validate_bits(activation_bits)
    validate_quantized_weight(weight)
    x = np.asarray(x)
    if x.ndim < 1:
        raise ValueError(f"activations must have at least one dimension, got {x.shape}")
    if not np.issubdtype(x.dtype, np.floating):
        raise TypeError(f"activations must be floating point, got {x.dtype}")
    if x.shape[-1] != weight.original_in_features:
        raise ValueError(
            f"activation K={x.shape[-1]} does not match weight K={weight.original_in_features}")
    flat = x.reshape((-1, x.shape[-1])).astype(F32)
    padded = np.zeros((flat.shape[0], weight.padded_in_features), dtype=F32)
    padded[:, : flat.shape[1]] = flat
    g = weight.group_size
    x_codes, x_scales = dynamic_group_quantize(padded, activation_bits, g)
    w_codes = unpacked_codes(weight).reshape((-1, g, weight.codes.shape[-1]))
    w_scales = weight.scales.astype(F32)
    n_groups = w_codes.shape[0]
    out = None
    accs = []
    for gi in range(n_groups):
        acc = int_matmul(x_codes[:, gi, :], w_codes[gi])
        scaled = acc.astype(F32) * x_scales[:, gi, None] * w_scales[gi][None, :]
        out = scaled if out is None else (out + scaled).astype(F32)
        if return_parts:
            accs.append(acc)
    out = out.reshape((*x.shape[:-1], w_codes.shape[-1])).astype(F32)
    if return_parts:
        return out, x_codes, x_scales, np.stack(accs, axis=1)
    return out


def quantized_frozen_linear(x, weight: GroupQuantizedWeight, *, activation_bits: int = 8):
    """quantized_lora.py:257-272 with a bf16 activation dtype."""
    return bf16_round(quantized_frozen_linear_f32(x, weight, activation_bits=activation_bits))


def quantized_lora_linear_f32(x, weight: GroupQuantizedWeight, lora_a, lora_b, lora_scaling,
                              *, activation_bits: int = 8):
    """Pre-cast value of quantized_lora.py:275-304: base + ((x@A)@B) * s, all float32."""
    validate_quantized_weight(weight)
    x = np.asarray(x)
    lora_a = np.asarray(lora_a)
    lora_b = np.asarray(lora_b)
    if lora_a.ndim != 2 or lora_b.ndim != 2:
        raise ValueError("lora_a and lora_b must both be rank-two")
    if lora_a.shape != (weight.original_in_features, lora_b.shape[0]):
        raise ValueError(
            f"incompatible LoRA shapes: A={lora_a.shape}, B={lora_b.shape}, "
            f"weight K={weight.original_in_features}")
    if lora_b.shape[1] != weight.codes.shape[-1]:
        raise ValueError(
            f"LoRA output N={lora_b.shape[1]} does not match weight N={weight.codes.shape[-1]}")
    scaling = np.asarray(lora_scaling, dtype=F32)
    if scaling.ndim != 0:
        raise ValueError(f"lora_scaling must be scalar, got {scaling.shape}")
    base = quantized_frozen_linear_f32(x, weight, activation_bits=activation_bits)
    flat = x.reshape((-1, x.shape[-1])).astype(F32)
    z = np.matmul(flat, lora_a.astype(F32), dtype=F32)
    low = np.matmul(z, lora_b.astype(F32), dtype=F32).reshape(base.shape)
    return (base + low * scaling).astype(F32)


def quantized_lora_linear(x, weight, lora_a, lora_b, lora_scaling, *, activation_bits: int = 8):
    """quantized_lora.py:400-453: exactly one bf16 cast after the float32 epilogue."""
    return bf16_round(quantized_lora_linear_f32(x, weight, lora_a, lora_b, lora_scaling,
                                                activation_bits=activation_bits))


# ---------------------------------------------------------------------------
# multi-adapter LoRA (skyrl/tx/layers/lora.py:118-157) in the float32-epilogue rule
# ---------------------------------------------------------------------------

def lora_delta_multi(x, lora_a, lora_b, lora_scaling, adapter_indices) -> np.ndarray:
    """Per-row adapter LoRA delta ((x @ A[i]) @ B[i]) * s[i] in float32.

    Routing follows lora.py:142-157 (rows grouped by adapter, two ragged products,
    scaling gathered per row); arithmetic follows the float32 rule of
    quantized_lora.py:300-304.  ``adapter_indices`` is one int per *row*.
    """
    x = np.asarray(x, dtype=F32)
    a = np.asarray(lora_a, dtype=F32)
    b = np.asarray(lora_b, dtype=F32)
    s = np.asarray(lora_scaling, dtype=F32)
    idx = np.asarray(adapter_indices)
    if a.ndim != 3 or b.ndim != 3:
        raise ValueError("multi-adapter lora_a/lora_b must be rank-three")
    if idx.shape != (x.shape[0],):
        raise ValueError("adapter_indices must hold one entry per row")
    if idx.size and (idx.min() < 0 or idx.max() >= a.shape[0]):
        raise ValueError("adapter index out of range")
    out = np.zeros((x.shape[0], b.shape[2]), dtype=F32)
    for adapter in np.unique(idx):
        rows = np.nonzero(idx == adapter)[0]
        z = np.matmul(x[rows], a[adapter], dtype=F32)
        out[rows] = np.matmul(z, b[adapter], dtype=F32) * s[adapter]
    return out


def quantized_lora_linear_multi_f32(x, weight, lora_a, lora_b, lora_scaling, adapter_indices,
                                    residual=None):
    """base + per-row LoRA delta (+ residual) in one float32 epilogue."""
    base = quantized_frozen_linear_f32(x, weight)
    out = (base + lora_delta_multi(x, lora_a, lora_b, lora_scaling, adapter_indices)).astype(F32)
    if residual is not None:
        out = (out + np.asarray(residual, dtype=F32)).astype(F32)
    return out


def quantized_lora_linear_multi(x, weight, lora_a, lora_b, lora_scaling, adapter_indices,
                                residual=None):
    """Single bf16 cast of ``quantized_lora_linear_multi_f32``.

    With ``residual`` this is the down-projection variant: the order follows the
    scalar HIP specification rocm/compile_probes/down_lora_residual_gfx1100.hip:120-123
    (float32 accumulate, += s*lora, += residual, one bf16 store).
    """
    return bf16_round(quantized_lora_linear_multi_f32(x, weight, lora_a, lora_b, lora_scaling,
                                                      adapter_indices, residual))


# ---------------------------------------------------------------------------
# backward of the quantized LoRA linear (quantized_lora.py:337-394)
# ---------------------------------------------------------------------------

def _mm64(a, b) -> np.ndarray:
    """float32 matrix product evaluated with float64 accumulation and rounded once.

    The reference contracts in float32 through XLA, whose summation order is not
    available here; the float64 sum is the order-free value every float32 order
    approximates (PARITY UNPINNED in the last float32 bits, far inside the bf16 gate).
    """
    return np.matmul(np.asarray(a, dtype=np.float64), np.asarray(b, dtype=np.float64)).astype(F32)


def pullback_weight(weight: GroupQuantizedWeight, relaxed: bool) -> np.ndarray:
    """[K, N] weight the input pull-back contracts with: float32 ``codes * scales``
    (quantized_lora.py:370) or, relaxed, that product rounded to bf16 per element, the policy of
    the ROCm kernel's W8A16 pull-back (skyrl/tx/kernels/rocm/w8a8_lora.py:326-330)."""
    wdeq = dequantize_frozen_weight(weight)[: weight.original_in_features]
    return bf16_round(wdeq) if relaxed else wdeq


def quantized_lora_linear_bwd_f32(x, weight: GroupQuantizedWeight, lora_a, lora_b, lora_scaling, dy,
                                  relaxed_weight: bool = False):
    """Float32 cotangents (dx, dA, dB, dscaling) of quantized_lora.py:337-394.

    Straight-through base: ``dx_base = dy @ (codes * scales).T`` (:361-378), the
    activation quantizer has no derivative of its own.  ``r = (dy @ B.T) * s`` (:352),
    ``dx = dx_base + r @ A.T`` (:379), ``dA = x.T @ r`` (:380), ``dB = ((x @ A).T @ dy) * s``
    (:381), ``dscaling = sum(dy * ((x @ A) @ B))`` (:382-383).
    """
    validate_quantized_weight(weight)
    x = np.asarray(x, dtype=F32)
    dy = np.asarray(dy, dtype=F32)
    a = np.asarray(lora_a, dtype=F32)
    b = np.asarray(lora_b, dtype=F32)
    s = F32(np.asarray(lora_scaling, dtype=F32).reshape(()))
    flat = x.reshape((-1, x.shape[-1]))
    dyf = dy.reshape((-1, dy.shape[-1]))
    if flat.shape[0] != dyf.shape[0]:
        raise ValueError("x and dy must have the same row domain")
    z = _mm64(flat, a)
    r = (_mm64(dyf, b.T) * s).astype(F32)
    wdeq = pullback_weight(weight, relaxed_weight)
    dx = (_mm64(dyf, wdeq.T) + _mm64(r, a.T)).astype(F32)
    da = _mm64(flat.T, r)
    db = (_mm64(z.T, dyf) * s).astype(F32)
    dscaling = F32(np.sum(dyf.astype(np.float64) * np.matmul(z.astype(np.float64), b.astype(np.float64))))
    return dx.reshape(x.shape), da, db, dscaling


def quantized_lora_linear_bwd(x, weight, lora_a, lora_b, lora_scaling, dy, relaxed_weight: bool = False):
    """Cotangents cast as the reference casts them (quantized_lora.py:384-391): dx to the
    activation dtype, dA/dB to the LoRA dtype (both bf16 here), dscaling to float32."""
    dx, da, db, ds = quantized_lora_linear_bwd_f32(x, weight, lora_a, lora_b, lora_scaling, dy, relaxed_weight)
    return bf16_round(dx), bf16_round(da), bf16_round(db), ds


def quantized_lora_linear_multi_bwd_f32(x, weight, lora_a, lora_b, lora_scaling, adapter_indices, dy,
                                        relaxed_weight: bool = False):
    """Per-row adapters: the cotangent of ``quantized_lora_linear_multi_f32``.

    Rows of adapter ``g`` contribute to ``dA[g]``, ``dB[g]``, ``dscaling[g]`` only (the
    derivative of the grouped products of skyrl/tx/layers/lora.py:142-157); adapters no row
    names get zeros.  The base term is shared.
    """
    x = np.asarray(x, dtype=F32)
    dy = np.asarray(dy, dtype=F32)
    a = np.asarray(lora_a, dtype=F32)
    b = np.asarray(lora_b, dtype=F32)
    s = np.asarray(lora_scaling, dtype=F32)
    idx = np.asarray(adapter_indices)
    if a.ndim != 3 or b.ndim != 3 or s.shape != (a.shape[0],):
        raise ValueError("multi-adapter lora_a/lora_b must be rank-three with one scaling each")
    if x.ndim != 2 or idx.shape != (x.shape[0],) or dy.shape[0] != x.shape[0]:
        raise ValueError("x, dy are [rows, .] with one adapter index per row")
    wdeq = pullback_weight(weight, relaxed_weight)
    dx = _mm64(dy, wdeq.T)
    da = np.zeros_like(a)
    db = np.zeros_like(b)
    ds = np.zeros_like(s)
    for g in np.unique(idx):
        rows = np.nonzero(idx == g)[0]
        z = _mm64(x[rows], a[g])
        r = (_mm64(dy[rows], b[g].T) * s[g]).astype(F32)
        dx[rows] = (dx[rows] + _mm64(r, a[g].T)).astype(F32)
        da[g] = _mm64(x[rows].T, r)
        db[g] = (_mm64(z.T, dy[rows]) * s[g]).astype(F32)
        ds[g] = F32(np.sum(dy[rows].astype(np.float64) * np.matmul(z.astype(np.float64), b[g].astype(np.float64))))
    return dx, da, db, ds


def quantized_lora_linear_multi_bwd(x, weight, lora_a, lora_b, lora_scaling, adapter_indices, dy,
                                    relaxed_weight: bool = False):
    dx, da, db, ds = quantized_lora_linear_multi_bwd_f32(x, weight, lora_a, lora_b, lora_scaling,
                                                         adapter_indices, dy, relaxed_weight)
    return bf16_round(dx), bf16_round(da), bf16_round(db), ds


# ---------------------------------------------------------------------------
# RMSNorm -> gate/up -> SwiGLU (bf16_rms_gate_up_lora_swiglu.py:277-330)
# ---------------------------------------------------------------------------

def rms_norm(x, gamma, eps: float = 1e-6) -> np.ndarray:
    """bf16(x * rsqrt(mean(x^2) + eps) * gamma); bf16_rms_gate_up_lora_swiglu.py:299-303.

    ``gamma`` is the float32 multiplier: ``1 + delta`` for the Qwen3.5 flavour
    (qwen3_5.py:269-278) or the plain weight for Qwen3 (layers/layernorm.py:22-24).
    mean = float32(sum in float64 / K); rsqrt = 1 / sqrt, both IEEE float32.
    """
    x = np.asarray(x, dtype=F32)
    gamma = np.asarray(gamma, dtype=F32)
    k = x.shape[-1]
    ssq = np.sum(x.astype(np.float64) * x.astype(np.float64), axis=-1, keepdims=True)
    var = (ssq / np.float64(k)).astype(F32)
    inv = (F32(1.0) / np.sqrt((var + F32(eps)).astype(F32))).astype(F32)
    normalized = (x * inv).astype(F32)
    return bf16_round((normalized * gamma).astype(F32))


def silu(v) -> np.ndarray:
    """x * logistic(x) in float32 (jax.nn.silu on an f32 operand)."""
    v = np.asarray(v, dtype=F32)
    with np.errstate(over="ignore"):
        sig = (F32(1.0) / (F32(1.0) + np.exp(-v).astype(F32))).astype(F32)
    return (v * sig).astype(F32)


def swiglu_from_interleaved(fused_bf16) -> np.ndarray:
    """bf16(silu(gate.f32) * up.f32) with gate = even, up = odd columns.

    Kernel rule of bf16_rms_gate_up_lora_swiglu.py:277-292 and
    bf16_rms_gate_up_lora_swiglu_contiguous.py:535-538.
    """
    fused = np.asarray(fused_bf16, dtype=F32)
    gate = fused[..., 0::2]
    up = fused[..., 1::2]
    return bf16_round((silu(gate) * up).astype(F32))


def w8a8_rms_gate_up_lora_swiglu(x, gamma, weight: GroupQuantizedWeight, lora_a, lora_b,
                                 lora_scaling, adapter_indices, eps: float = 1e-6,
                                 return_stages: bool = False):
    """Composite oracle for the fused W8A8 MLP-up stage.

    n = rms_norm(x) (bf16) -> per-token A8 quantization of n -> int GEMM + f32
    dequant -> + s[idx] * ((n @ A[idx]) @ B[idx]) in f32 -> one bf16 cast (fused)
    -> adjacent (gate, up) pairs -> bf16(silu(gate) * up).
    """
    n = rms_norm(x, gamma, eps)
    fused_f32 = quantized_lora_linear_multi_f32(n, weight, lora_a, lora_b, lora_scaling,
                                                adapter_indices)
    fused = bf16_round(fused_f32)
    product = swiglu_from_interleaved(fused)
    if return_stages:
        return product, {"normalized": n, "fused_f32": fused_f32, "fused": fused}
    return product


# ---------------------------------------------------------------------------
# backward of RMSNorm -> gate/up -> SwiGLU
# (rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:541-574, 643-689)
# ---------------------------------------------------------------------------

def swiglu_pullback_interleaved(fused_bf16, d_product) -> np.ndarray:
    """bf16 cotangent of the interleaved projection; float32 operations in the order of
    bf16_rms_gate_up_lora_swiglu_contiguous.py:541-553:
    d_up = c * (g * sig), d_gate = (c * u) * sig + (g * (c * u)) * (sig * (1 - sig)).
    """
    fused = np.asarray(fused_bf16, dtype=F32)
    gate = fused[..., 0::2]
    up = fused[..., 1::2]
    c = np.asarray(d_product, dtype=F32).reshape(gate.shape)
    with np.errstate(over="ignore"):
        sig = (F32(1.0) / (F32(1.0) + np.exp(-gate).astype(F32))).astype(F32)
    d_up = (c * (gate * sig).astype(F32)).astype(F32)
    wc = (c * up).astype(F32)
    sprime = (sig * (F32(1.0) - sig).astype(F32)).astype(F32)
    d_gate = ((wc * sig).astype(F32) + ((gate * wc).astype(F32) * sprime).astype(F32)).astype(F32)
    out = np.empty(fused.shape, dtype=F32)
    out[..., 0::2] = d_gate
    out[..., 1::2] = d_up
    return bf16_round(out)


def rms_norm_pullback(x, gamma, d_normalized, eps: float = 1e-6) -> np.ndarray:
    """bf16 cotangent of x through ``rms_norm``; bf16_rms_gate_up_lora_swiglu_contiguous.py:556-574.

    p = dn * gamma; den = mean(x^2) + eps and inv = 1 / sqrt(den) as in ``rms_norm``;
    t = (sum_k x p) * (-0.5 * (inv / den)) / K; dx = bf16((p * inv + x * t) + t * x).
    The row sum is taken in float64 and rounded once (the reference's float32 reduction order is
    XLA's: PARITY UNPINNED in its last bits).
    """
    x = np.asarray(x, dtype=F32)
    gamma = np.asarray(gamma, dtype=F32)
    dn = np.asarray(d_normalized, dtype=F32)
    k = x.shape[-1]
    ssq = np.sum(x.astype(np.float64) * x.astype(np.float64), axis=-1, keepdims=True)
    den = ((ssq / np.float64(k)).astype(F32) + F32(eps)).astype(F32)
    inv = (F32(1.0) / np.sqrt(den)).astype(F32)
    p = (dn * gamma).astype(F32)
    ic = np.sum(x.astype(np.float64) * p.astype(np.float64), axis=-1, keepdims=True).astype(F32)
    dc = (ic * (F32(-0.5) * (inv / den).astype(F32)).astype(F32)).astype(F32)
    t = (dc / F32(k)).astype(F32)
    xt = (x * t).astype(F32)
    return bf16_round((((p * inv).astype(F32) + xt).astype(F32) + xt).astype(F32))


def w8a8_rms_gate_up_lora_swiglu_bwd(x, gamma, weight: GroupQuantizedWeight, lora_a, lora_b, lora_scaling,
                                     adapter_indices, d_product, eps: float = 1e-6,
                                     relaxed_weight: bool = True, return_stages: bool = False):
    """Cotangents (dx, dA, dB, dscaling) of ``w8a8_rms_gate_up_lora_swiglu``.

    The structure of bf16_rms_gate_up_lora_swiglu_contiguous.py:643-689 (SwiGLU pull-back on the
    saved bf16 projection, the projection's pull-back on the bf16 normalized rows, the RMSNorm
    pull-back) with the quantized projection's own rule in the middle
    (``quantized_lora_linear_multi_bwd``: straight-through quantizer, LoRA terms in float32, one
    cast per cotangent).
    """
    product, stages = w8a8_rms_gate_up_lora_swiglu(x, gamma, weight, lora_a, lora_b, lora_scaling,
                                                   adapter_indices, eps, return_stages=True)
    d_fused = swiglu_pullback_interleaved(stages["fused"], d_product)
    dn, da, db, ds = quantized_lora_linear_multi_bwd(stages["normalized"], weight, lora_a, lora_b, lora_scaling,
                                                     adapter_indices, d_fused, relaxed_weight)
    dx = rms_norm_pullback(x, gamma, dn, eps)
    if return_stages:
        return (dx, da, db, ds), {"d_fused": d_fused, "d_normalized": dn, **stages}
    return dx, da, db, ds


# ---------------------------------------------------------------------------
# fused-projection interleave (skyrl/tx/layers/lora.py:325-351)
# ---------------------------------------------------------------------------

def fuse(*arrays, group_sizes) -> np.ndarray:
    assert len(arrays) == len(group_sizes)
    batch = arrays[0].shape[:-1]
    num_groups = arrays[0].shape[-1] // group_sizes[0]
    parts = []
    for arr, g in zip(arrays, group_sizes):
        assert arr.shape[-1] == num_groups * g
        parts.append(np.asarray(arr).reshape(*batch, num_groups, g))
    return np.concatenate(parts, axis=-1).reshape(*batch, -1)


def split(fused, group_sizes):
    fused = np.asarray(fused)
    batch, total = fused.shape[:-1], fused.shape[-1]
    gs = sum(group_sizes)
    assert total % gs == 0
    num_groups = total // gs
    view = fused.reshape(*batch, num_groups, gs)
    out, offset = [], 0
    for g in group_sizes:
        out.append(view[..., offset:offset + g].reshape(*batch, num_groups * g))
        offset += g
    return tuple(out)


# ---------------------------------------------------------------------------
# routing helpers (skyrl/tx/layers/util.py:8-87)
# ---------------------------------------------------------------------------

def prepare_routing(tokens, indices, num_groups: int, adapter_indices=None):
    """util.py:66-87: stable argsort by group, bincount, inverse permutation."""
    indices = np.asarray(indices)
    sort_indices = np.argsort(indices, kind="stable")
    sorted_tokens = np.asarray(tokens)[sort_indices]
    sorted_adapters = None if adapter_indices is None else np.asarray(adapter_indices)[sort_indices]
    group_sizes = np.bincount(indices, minlength=num_groups)[:num_groups]
    unsort = np.argsort(sort_indices, kind="stable")
    return sorted_tokens, group_sizes, unsort, sorted_adapters


def ragged_dot(lhs, rhs, group_sizes, group_offset=None) -> np.ndarray:
    """util.py:8-59: rows of group g are multiplied by rhs[g]; with ``group_offset``
    rhs holds groups [offset, offset + g_local) and rows of other groups give zero.
    Rows beyond sum(group_sizes) give zero (lax.ragged_dot semantics)."""
    lhs = np.asarray(lhs, dtype=F32)
    rhs = np.asarray(rhs, dtype=F32)
    group_sizes = np.asarray(group_sizes)
    offset = 0 if group_offset is None else int(np.asarray(group_offset).reshape(-1)[0])
    out = np.zeros((lhs.shape[0], rhs.shape[2]), dtype=F32)
    starts = np.concatenate(([0], np.cumsum(group_sizes)))
    for local in range(rhs.shape[0]):
        g = local + offset
        if g >= len(group_sizes):
            break
        r0, r1 = int(starts[g]), int(starts[g + 1])
        if r1 > r0:
            out[r0:r1] = np.matmul(lhs[r0:r1], rhs[local], dtype=F32)
    return out


# ---------------------------------------------------------------------------
# MoE expert MLP (skyrl/tx/models/qwen3.py:172-210, layers/lora.py:394-444)
# ---------------------------------------------------------------------------

def moe_route(router_logits, top_k: int, norm_topk_prob: bool = True):
    """softmax -> top_k -> renormalise; qwen3.py:175-178.  Ties pick the lower index."""
    logits = np.asarray(router_logits, dtype=F32)
    shifted = logits - np.max(logits, axis=-1, keepdims=True)
    e = np.exp(shifted).astype(F32)
    probs = (e / np.sum(e, axis=-1, keepdims=True, dtype=F32)).astype(F32)
    order = np.argsort(-probs, axis=-1, kind="stable")[:, :top_k]
    weights = np.take_along_axis(probs, order, axis=-1)
    if norm_topk_prob:
        weights = (weights / np.sum(weights, axis=-1, keepdims=True, dtype=F32)).astype(F32)
    return weights.astype(F32), order.astype(np.int32)


def grouped_quantized_lora_linear_f32(x_sorted, group_sizes, weights, lora_a, lora_b, scaling):
    """Per-expert quantized LoRA linear over contiguous row groups, float32 pre-cast.

    ``weights`` is a list of per-expert GroupQuantizedWeight; ``lora_a``/``lora_b``
    are [E, K, r] / [E, r, N]; ``scaling`` a float32 scalar (lora.py:433-444 with a
    single adapter; expert e's rows use A[e], B[e]).
    """
    x_sorted = np.asarray(x_sorted, dtype=F32)
    n_out = weights[0].codes.shape[1]
    out = np.zeros((x_sorted.shape[0], n_out), dtype=F32)
    starts = np.concatenate(([0], np.cumsum(np.asarray(group_sizes))))
    for e, w in enumerate(weights):
        r0, r1 = int(starts[e]), int(starts[e + 1])
        if r1 > r0:
            out[r0:r1] = quantized_lora_linear_f32(x_sorted[r0:r1], w, lora_a[e], lora_b[e], scaling)
    return out


def moe_combine(expert_out, unsort, weights) -> np.ndarray:
    """bf16(sum_j f32(expert_out[unsort[t k + j]]) * weights[t, j]); qwen3.py:205-207 with the products
    and the sum over the choices in float32, choice order, one cast."""
    weights = np.asarray(weights, dtype=F32)
    t, top_k = weights.shape
    per_tok = np.asarray(expert_out, dtype=F32)[np.asarray(unsort)].reshape(t, top_k, -1)
    return bf16_round(np.sum(per_tok * weights[..., None], axis=1, dtype=F32))


def moe_expert_mlp(hidden, router_logits, top_k, gate_up_weights, down_weights,
                   gate_up_a, gate_up_b, down_a, down_b, scaling, return_stages: bool = False):
    """Composite oracle for the grouped W8A8 + LoRA expert MLP.

    Routing as in qwen3.py:172-210; gate/up are fused per expert in the adjacent
    (gate, up) column interleave; every stage boundary is one bf16 cast; the
    combine ``sum_k down * w_k`` is evaluated in float32 and cast once.
    """
    hidden = np.asarray(hidden, dtype=F32)
    n_experts = len(gate_up_weights)
    weights, selected = moe_route(router_logits, top_k)
    expanded = np.repeat(hidden, top_k, axis=0)
    x_sorted, group_sizes, unsort, _ = prepare_routing(expanded, selected.ravel(), n_experts)
    fused = bf16_round(grouped_quantized_lora_linear_f32(
        x_sorted, group_sizes, gate_up_weights, gate_up_a, gate_up_b, scaling))
    act = swiglu_from_interleaved(fused)
    down = bf16_round(grouped_quantized_lora_linear_f32(
        act, group_sizes, down_weights, down_a, down_b, scaling))
    out = moe_combine(down, unsort, weights)
    if return_stages:
        return out, {"group_sizes": group_sizes, "unsort": unsort, "x_sorted": x_sorted,
                     "fused": fused, "act": act, "down": down, "weights": weights,
                     "selected": selected}
    return out


# ---------------------------------------------------------------------------
# pull-back of the expert MLP: the derivative of qwen3.py:172-210, written out
# ---------------------------------------------------------------------------

def moe_combine_bwd(d_out, expert_out, unsort, weights):
    """Cotangents of ``moe_combine`` in its two operands: d_expert_out[unsort[t k + j]] =
    bf16(d_out[t] * w[t, j]) and d_w[t, j] = sum_c expert_out[unsort[t k + j], c] * d_out[t, c]
    (float32 products, summed in float64 and rounded once)."""
    d_out = np.asarray(d_out, dtype=F32)
    expert_out = np.asarray(expert_out, dtype=F32)
    w = np.asarray(weights, dtype=F32)
    t, k = w.shape
    rows = np.asarray(unsort).reshape(t, k)
    d_expert = np.zeros_like(expert_out)
    d_w = np.zeros_like(w)
    for j in range(k):
        d_expert[rows[:, j]] = bf16_round((d_out * w[:, j:j + 1]).astype(F32))
        d_w[:, j] = np.sum((expert_out[rows[:, j]] * d_out).astype(F32).astype(np.float64), axis=1).astype(F32)
    return d_expert, d_w


def moe_route_bwd(router_logits, selected, d_weights, norm_topk_prob: bool = True) -> np.ndarray:
    """Cotangent of the router logits through softmax -> (fixed) top-k selection -> renormalisation
    (qwen3.py:175-178), float64 inside, float32 out."""
    logits = np.asarray(router_logits, dtype=np.float64)
    sel = np.asarray(selected)
    dw = np.asarray(d_weights, dtype=np.float64)
    z = logits - logits.max(axis=-1, keepdims=True)
    p = np.exp(z)
    p /= p.sum(axis=-1, keepdims=True)
    ps = np.take_along_axis(p, sel, axis=1)
    if norm_topk_prob:
        tot = ps.sum(axis=-1, keepdims=True)
        w = ps / tot
        dps = (dw - np.sum(dw * w, axis=-1, keepdims=True)) / tot
    else:
        dps = dw
    dp = np.zeros_like(p)
    np.put_along_axis(dp, sel, dps, axis=1)
    return (p * (dp - np.sum(p * dp, axis=-1, keepdims=True))).astype(F32)


def moe_expert_mlp_bwd(hidden, router_logits, top_k, gate_up_weights, down_weights, gate_up_a, gate_up_b,
                       down_a, down_b, scaling, d_out, relaxed_weight: bool = True):
    """Cotangents of ``moe_expert_mlp``: the chain combine -> grouped down -> SwiGLU -> grouped gate/up ->
    gather written backwards, every grouped projection under ``quantized_lora_linear_bwd`` per expert,
    every stage boundary one bf16 cast, the scatter-add of the gather summed in float32 in choice
    order.  ``scaling`` is one float32 scalar shared by all experts and both projections.  Returns a
    dict: d_hidden, d_router_logits, d_gate_up_a/b, d_down_a/b, d_scaling."""
    hidden = np.asarray(hidden, dtype=F32)
    _, st = moe_expert_mlp(hidden, router_logits, top_k, gate_up_weights, down_weights, gate_up_a, gate_up_b,
                           down_a, down_b, scaling, return_stages=True)
    sizes, unsort = st["group_sizes"], st["unsort"]
    d_down, d_w = moe_combine_bwd(d_out, st["down"], unsort, st["weights"])
    starts = np.concatenate(([0], np.cumsum(sizes)))

    def grouped_bwd(x, dy, weights, a, b):
        dx = np.zeros_like(x)
        da, db = np.zeros_like(a), np.zeros_like(b)
        ds = F32(0.0)
        for e, w in enumerate(weights):
            r0, r1 = int(starts[e]), int(starts[e + 1])
            if r1 > r0:
                dx[r0:r1], da[e], db[e], dse = quantized_lora_linear_bwd(x[r0:r1], w, a[e], b[e], scaling, dy[r0:r1],
                                                                         relaxed_weight)
                ds = F32(ds + F32(dse))
        return dx, da, db, ds

    d_act, d_da, d_db, ds_dn = grouped_bwd(st["act"], d_down, down_weights, np.asarray(down_a, F32), np.asarray(down_b, F32))
    d_fused = swiglu_pullback_interleaved(st["fused"], d_act)
    d_xs, d_ga, d_gb, ds_gu = grouped_bwd(st["x_sorted"], d_fused, gate_up_weights, np.asarray(gate_up_a, F32),
                                          np.asarray(gate_up_b, F32))
    d_hidden = moe_combine(d_xs, unsort, np.ones_like(st["weights"]))
    return {"d_hidden": d_hidden, "d_router_logits": moe_route_bwd(router_logits, st["selected"], d_w),
            "d_weights": d_w, "d_gate_up_a": d_ga, "d_gate_up_b": d_gb, "d_down_a": d_da, "d_down_b": d_db,
            "d_scaling": F32(ds_dn + ds_gu), "d_down": d_down, "d_act": d_act, "d_fused": d_fused, "stages": st}


# ---------------------------------------------------------------------------
# numerical gate (rocm/probe_w8a8_lora_forward.py:186-189, 1291-1369)
# ---------------------------------------------------------------------------

MAX_RELATIVE_L2_ERROR = 0.01
MIN_COSINE_SIMILARITY = 0.9999
MAX_ABSOLUTE_ERROR = 0.25


def numerical_gate(candidate, expected) -> dict:
    c = np.asarray(candidate, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    diff = c - e
    den = max(float(np.linalg.norm(e)), 1e-12)
    rel_l2 = float(np.linalg.norm(diff)) / den
    cos_den = float(np.linalg.norm(c)) * float(np.linalg.norm(e))
    cosine = float(np.dot(c, e)) / cos_den if cos_den > 0 else (1.0 if not diff.any() else 0.0)
    max_abs = float(np.max(np.abs(diff))) if diff.size else 0.0
    finite = bool(np.all(np.isfinite(c)))
    passed = finite and rel_l2 < MAX_RELATIVE_L2_ERROR and cosine >= MIN_COSINE_SIMILARITY \
        and max_abs <= MAX_ABSOLUTE_ERROR
    return {"relative_l2": rel_l2, "cosine": cosine, "max_abs": max_abs, "finite": finite,
            "passed": passed}


def within_tolerance(candidate, expected, atol: float = 2e-2, rtol: float = 1e-2) -> np.ndarray:
    """Elementwise |a - b| <= atol + rtol * |b| (the bf16 output criterion)."""
    c = np.asarray(candidate, dtype=np.float64)
    e = np.asarray(expected, dtype=np.float64)
    return np.abs(c - e) <= atol + rtol * np.abs(e)
