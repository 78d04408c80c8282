"""jax.ffi registration and call wrappers for the W8A8 kernels (XLA typed FFI).

The JAX side of the drop-in: the same function names as the torch host mirror in
``w8a8_lora.py`` but taking/returning ``jax.Array``.  Registration follows the
reference's ``skyrl/tx/kernels/rocm/gdn_ffi_smoke.py:281-353``: ``ctypes.CDLL`` on the
shim library, ``handler.restype = c_void_p``, ``jax.ffi.pycapsule``,
``jax.ffi.register_ffi_target(name, capsule, platform="ROCM", api_version=1)``, the
library kept alive for the life of the process, one registration per process under a
lock.  Calls use ``jax.ffi.ffi_call(..., vmap_method="sequential",
custom_call_api_version=4)`` with row-major layouts (gdn_ffi_smoke.py:401-414).

JAX and jaxlib are imported lazily: this module imports everywhere, the functions
raise ``RuntimeError`` where JAX or the shim library (``libmi355_w8a8_ffi.so``, built
only where jaxlib's headers exist) is missing.
"""

from __future__ import annotations

import ctypes
import threading
from pathlib import Path

from ... import _native

FFI_LIB_PATH = Path(_native.LIB_PATH).with_name("libmi355_w8a8_ffi.so")
TARGETS = ("mi355_w8a8_ffi_forward_v1", "mi355_w8a8_ffi_quantize_rows_v1", "mi355_w8a8_ffi_pack_weight_v1",
           "mi355_w8a8_ffi_backward_v1", "mi355_w8a8_ffi_swiglu_bwd_v1", "mi355_w8a8_ffi_rms_norm_bwd_v1",
           "mi355_w8a8_ffi_moe_route_v1", "mi355_w8a8_ffi_moe_dispatch_v1", "mi355_w8a8_ffi_moe_combine_v1",
           "mi355_w8a8_ffi_grouped_v1", "mi355_w8a8_ffi_qkv_split_norm_rope_v1", "mi355_w8a8_ffi_gq_pack_weight_v1",
           "mi355_w8a8_ffi_gq_linear_v1", "mi355_w8a8_ffi_grouped_bwd_v1", "mi355_w8a8_ffi_qkv_split_norm_rope_bwd_v1",
           "mi355_w8a8_ffi_delta_rms_norm_bwd_v1", "mi355_w8a8_ffi_moe_route_bwd_v1", "mi355_w8a8_ffi_moe_combine_bwd_v1")
_ROCM_PLATFORM = "ROCM"
_REGISTRATION_API_VERSION = 1
_CUSTOM_CALL_API_VERSION = 4

_lock = threading.Lock()
_registered = False
_lifetime_handles: list = []


def _import_jax():
    try:
        import jax  # noqa: PLC0415
    except ImportError as error:  # pragma: no cover - depends on the environment
        raise RuntimeError("the XLA FFI route needs jax/jaxlib, which is not installed") from error
    return jax


def _load_cdll(path: Path):
    return ctypes.CDLL(str(path), mode=ctypes.RTLD_LOCAL)


def register(jax_module=None) -> tuple[str, ...]:
    """Register the FFI targets once per process; returns the target names."""
    global _registered
    jax = jax_module or _import_jax()
    ffi = getattr(jax, "ffi", None)
    if ffi is None or not all(callable(getattr(ffi, n, None)) for n in ("pycapsule", "register_ffi_target", "ffi_call")):
        raise RuntimeError("installed JAX does not expose the required typed-FFI API")
    with _lock:
        if _registered:
            return TARGETS
        if not FFI_LIB_PATH.exists():
            raise RuntimeError(f"{FFI_LIB_PATH} is missing: build it where jaxlib's xla/ffi headers are installed")
        # the C ABI library must be resident first: the shim links against it
        _lifetime_handles.append(ctypes.CDLL(str(_native.LIB_PATH), mode=ctypes.RTLD_GLOBAL))
        library = _load_cdll(FFI_LIB_PATH)
        _lifetime_handles.append(library)  # a capsule is a bare function pointer: never unload
        for name in TARGETS:
            try:
                handler = getattr(library, name)
            except AttributeError as error:
                raise RuntimeError(f"FFI library is missing its handler symbol {name}") from error
            handler.restype = ctypes.c_void_p
            handler.argtypes = (ctypes.c_void_p,)
            ffi.register_ffi_target(name, ffi.pycapsule(handler), platform=_ROCM_PLATFORM,
                                    api_version=_REGISTRATION_API_VERSION)
        _registered = True
        return TARGETS


def _row_major(ndim: int) -> tuple[int, ...]:
    return tuple(range(ndim - 1, -1, -1))


def _call(jax, name, result_specs, *operands, **attrs):
    call = jax.ffi.ffi_call(
        name, result_specs, has_side_effect=False, vmap_method="sequential",
        input_layouts=tuple(_row_major(o.ndim) for o in operands),
        output_layouts=tuple(_row_major(len(s.shape)) for s in result_specs),
        input_output_aliases=None, custom_call_api_version=_CUSTOM_CALL_API_VERSION)
    return call(*operands, **attrs)


def pack_weight(codes):
    """int8 [K, N] codes -> opaque uint8 packed weight (run once per weight, not per forward)."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k, n = codes.shape
    nbytes = int(_native.load().mi355_w8a8_packed_weight_bytes(k, n))
    (packed,) = _call(jax, TARGETS[2], (jax.ShapeDtypeStruct((nbytes,), jnp.uint8),), codes)
    return packed


def quantize_rows(x):
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    return _call(jax, TARGETS[1], (jax.ShapeDtypeStruct(x.shape, jnp.int8),
                                   jax.ShapeDtypeStruct(x.shape[:-1], jnp.float32)), x)


def forward(x, packed_weight, w_scales, lora_a=None, lora_b=None, lora_scaling=None, adapter_indices=None,
            rms_gamma=None, residual=None, *, swiglu: bool = False, eps: float = 1e-6, entry: int = 0):
    """W8A8 (+LoRA, +RMSNorm, +SwiGLU, +residual) forward as one XLA custom call."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k = x.shape[-1]
    n = w_scales.shape[-1]
    m = 1
    for d in x.shape[:-1]:
        m *= d
    empty = lambda dt, nd: jnp.zeros((0,) * nd, dt)
    a3 = empty(jnp.bfloat16, 3) if lora_a is None else (lora_a if lora_a.ndim == 3 else lora_a[None])
    b3 = empty(jnp.bfloat16, 3) if lora_b is None else (lora_b if lora_b.ndim == 3 else lora_b[None])
    n_ad = a3.shape[0]
    s1 = empty(jnp.float32, 1) if lora_a is None else jnp.broadcast_to(jnp.asarray(lora_scaling, jnp.float32), (n_ad,))
    idx = empty(jnp.int32, 1) if adapter_indices is None else adapter_indices.astype(jnp.int32).reshape(-1)
    gamma = empty(jnp.float32, 1) if rms_gamma is None else rms_gamma.astype(jnp.float32)
    res = empty(jnp.bfloat16, 2) if residual is None else residual.reshape(m, -1)
    n_out = n // 2 if swiglu else n
    ws = int(_native.load().mi355_w8a8_workspace_bytes(m, k, n, n_ad, a3.shape[2] if n_ad else 0, 1 if swiglu else 0))
    if ws == 0:
        raise ValueError(f"geometry M={m}, K={k}, N={n} is outside the native path")
    y, _ = _call(jax, TARGETS[0],
                 (jax.ShapeDtypeStruct((*x.shape[:-1], n_out), jnp.bfloat16), jax.ShapeDtypeStruct((ws,), jnp.uint8)),
                 x, packed_weight, w_scales.reshape(n).astype(jnp.float32), a3, b3, s1, idx, gamma, res,
                 swiglu=int(swiglu), rms_eps=float(eps), entry=int(entry))
    return y


def backward(x, dy, packed_weight, w_scales, lora_a=None, lora_b=None, lora_scaling=None, adapter_indices=None):
    """Cotangents of the plain linear as one XLA custom call: ``(dx, dA, dB, dscaling)`` (the LoRA
    entries are ``None`` without LoRA).  This is the body of the ``custom_vjp`` backward rule that
    replaces ``_quantized_lora_linear_bwd`` (skyrl/tx/kernels/quantized_lora.py:337-394)."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k = x.shape[-1]
    n = w_scales.shape[-1]
    m = 1
    for d in x.shape[:-1]:
        m *= d
    empty = lambda dt, nd: jnp.zeros((0,) * nd, dt)
    a3 = empty(jnp.bfloat16, 3) if lora_a is None else (lora_a if lora_a.ndim == 3 else lora_a[None])
    b3 = empty(jnp.bfloat16, 3) if lora_b is None else (lora_b if lora_b.ndim == 3 else lora_b[None])
    n_ad = a3.shape[0]
    rank = a3.shape[2] if n_ad else 0
    s1 = empty(jnp.float32, 1) if lora_a is None else jnp.broadcast_to(jnp.asarray(lora_scaling, jnp.float32), (n_ad,))
    idx = empty(jnp.int32, 1) if adapter_indices is None else adapter_indices.astype(jnp.int32).reshape(-1)
    ws = int(_native.load().mi355_w8a8_bwd_workspace_bytes(m, k, n, n_ad, rank, 0))
    if ws == 0:
        raise ValueError(f"geometry M={m}, K={k}, N={n} is outside the native backward")
    dx, da, db, ds, _ = _call(
        jax, TARGETS[3],
        (jax.ShapeDtypeStruct(x.shape, jnp.bfloat16), jax.ShapeDtypeStruct(a3.shape, jnp.bfloat16),
         jax.ShapeDtypeStruct(b3.shape, jnp.bfloat16), jax.ShapeDtypeStruct(s1.shape, jnp.float32),
         jax.ShapeDtypeStruct((ws,), jnp.uint8)),
        x, dy, packed_weight, w_scales.reshape(n).astype(jnp.float32), a3, b3, s1, idx)
    if lora_a is None:
        return dx, None, None, None
    if lora_a.ndim == 2:
        return dx, da[0], db[0], ds[0]
    return dx, da, db, ds


def grouped(x, packed_weights, w_scales, group_sizes, lora_a=None, lora_b=None, lora_scaling=None, *,
            swiglu: bool = False, x_row_map=None, x_row_repeat: int = 1):
    """Ragged per-group W8A8 (+LoRA, +SwiGLU) linear over rows sorted by group as one XLA custom call: the
    expert projection of ``LoRAExpert.__call__`` (skyrl/tx/layers/lora.py:394-444).  ``packed_weights`` holds
    the groups' packed weights back to back, ``w_scales`` is f32 [n_weights, N].  With ``x_row_map`` (the
    dispatch's sort indices) row i of the call is read from ``x[x_row_map[i] // x_row_repeat]``."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k = x.shape[-1]
    n = w_scales.shape[-1]
    n_groups = group_sizes.shape[0]
    empty = lambda dt, nd: jnp.zeros((0,) * nd, dt)
    a3 = empty(jnp.bfloat16, 3) if lora_a is None else lora_a
    b3 = empty(jnp.bfloat16, 3) if lora_b is None else lora_b
    rank = a3.shape[2] if lora_a is not None else 0
    s1 = (empty(jnp.float32, 1) if lora_a is None
          else jnp.broadcast_to(jnp.asarray(lora_scaling, jnp.float32), (n_groups,)))
    row_map = empty(jnp.int32, 1) if x_row_map is None else x_row_map.astype(jnp.int32).reshape(-1)
    m = row_map.shape[0] if x_row_map is not None else x.reshape(-1, k).shape[0]
    if x_row_map is not None and (x_row_repeat < 1 or x.reshape(-1, k).shape[0] * x_row_repeat < m):
        raise ValueError("x_row_map names more rows than x holds times x_row_repeat")
    n_out = n // 2 if swiglu else n
    ws = int(_native.load().mi355_w8a8_grouped_workspace_bytes(m, k, n, n_groups, rank, 1 if swiglu else 0))
    if ws == 0:
        raise ValueError(f"geometry M={m}, K={k}, N={n}, groups={n_groups} is outside the native path")
    y, _ = _call(jax, TARGETS[9],
                 (jax.ShapeDtypeStruct((m, n_out), jnp.bfloat16), jax.ShapeDtypeStruct((ws,), jnp.uint8)),
                 x.reshape(-1, k), packed_weights, w_scales.reshape(-1, n).astype(jnp.float32), a3, b3, s1,
                 group_sizes.astype(jnp.int32), row_map, swiglu=int(swiglu), x_row_repeat=int(x_row_repeat))
    return y


def qkv_split_norm_rope(fused, q_norm_weight, k_norm_weight, positions, *, num_query_heads: int, num_kv_heads: int,
                        head_dim: int, rotary_dim: int, rope_theta: float, eps: float = 1e-6):
    """Split / head RMSNorm / partial RoPE behind the fused QKV projection as one XLA custom call
    (skyrl/tx/kernels/qwen3_5_qkv_lora.py:266-286): returns ``(q, k, v, gate)``."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    width = num_query_heads * 2 * head_dim + 2 * num_kv_heads * head_dim
    if fused.shape[-1] != width:
        raise ValueError(f"fused projection must be [..., {width}]")
    lead = fused.shape[:-1]
    m = 1
    for d in lead:
        m *= d
    q, k, v, gate = _call(
        jax, TARGETS[10],
        (jax.ShapeDtypeStruct((m, num_query_heads, head_dim), jnp.bfloat16),
         jax.ShapeDtypeStruct((m, num_kv_heads, head_dim), jnp.bfloat16),
         jax.ShapeDtypeStruct((m, num_kv_heads, head_dim), jnp.bfloat16),
         jax.ShapeDtypeStruct((m, num_query_heads * head_dim), jnp.bfloat16)),
        fused.reshape(m, width), q_norm_weight.astype(jnp.float32), k_norm_weight.astype(jnp.float32),
        positions.astype(jnp.int32).reshape(m), rotary_dim=int(rotary_dim), rope_theta=float(rope_theta),
        rms_eps=float(eps))
    return (q.reshape(*lead, num_query_heads, head_dim), k.reshape(*lead, num_kv_heads, head_dim),
            v.reshape(*lead, num_kv_heads, head_dim), gate.reshape(*lead, num_query_heads * head_dim))


def gq_pack_weight(codes, weight_bits: int):
    """int8 [K_pad, N] group-scaled codes (4-bit codes one per byte) -> opaque uint8 packed weight."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k_pad, n = codes.shape
    nbytes = int(_native.load().mi355_w8a8_gq_packed_weight_bytes(k_pad, n, weight_bits))
    if nbytes == 0:
        raise ValueError(f"geometry K_pad={k_pad}, N={n}, W{weight_bits} is outside the native path")
    (packed,) = _call(jax, TARGETS[11], (jax.ShapeDtypeStruct((nbytes,), jnp.uint8),), codes,
                      weight_bits=int(weight_bits))
    return packed


def gq_linear(x, packed_weight, w_scales, *, group_size: int, weight_bits: int, activation_bits: int,
              lora_a=None, lora_b=None, lora_scaling=None, adapter_indices=None):
    """Group-scaled W4/W8 x A4/A8 (+LoRA) linear as one XLA custom call: the general form of
    ``_quantized_frozen_linear_f32`` (skyrl/tx/kernels/quantized_lora.py:215-304)."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k = x.shape[-1]
    n_grp, n = w_scales.shape
    m = 1
    for d in x.shape[:-1]:
        m *= d
    empty = lambda dt, nd: jnp.zeros((0,) * nd, dt)
    a3 = empty(jnp.bfloat16, 3) if lora_a is None else (lora_a if lora_a.ndim == 3 else lora_a[None])
    b3 = empty(jnp.bfloat16, 3) if lora_b is None else (lora_b if lora_b.ndim == 3 else lora_b[None])
    n_ad = a3.shape[0]
    s1 = empty(jnp.float32, 1) if lora_a is None else jnp.broadcast_to(jnp.asarray(lora_scaling, jnp.float32), (n_ad,))
    idx = empty(jnp.int32, 1) if adapter_indices is None else adapter_indices.astype(jnp.int32).reshape(-1)
    ws = int(_native.load().mi355_w8a8_gq_workspace_bytes(m, n_grp * group_size, group_size, n_ad,
                                                          a3.shape[2] if n_ad else 0))
    if ws == 0:
        raise ValueError(f"geometry M={m}, K_pad={n_grp * group_size}, group {group_size} is outside the native path")
    y, _ = _call(jax, TARGETS[12],
                 (jax.ShapeDtypeStruct((*x.shape[:-1], n), jnp.bfloat16), jax.ShapeDtypeStruct((ws,), jnp.uint8)),
                 x, packed_weight, w_scales.astype(jnp.float32), a3, b3, s1, idx, group_size=int(group_size),
                 weight_bits=int(weight_bits), activation_bits=int(activation_bits))
    return y


def swiglu_bwd(fused, d_product):
    """Cotangent of the fused gate/up projection from the cotangent of ``silu(gate) * up``
    (skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:541-574)."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    (d_fused,) = _call(jax, TARGETS[4], (jax.ShapeDtypeStruct(fused.shape, jnp.bfloat16),), fused, d_product)
    return d_fused


def rms_norm_bwd(x, gamma, d_normalized, *, eps: float = 1e-6):
    """Cotangent of the rows going into the RMSNorm prologue."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    (d_x,) = _call(jax, TARGETS[5], (jax.ShapeDtypeStruct(x.shape, jnp.bfloat16),), x, gamma.astype(jnp.float32),
                   d_normalized, eps=float(eps))
    return d_x


def moe_route(router_logits, top_k: int, norm_topk_prob: bool):
    """softmax / top-k (/ renormalisation) of the router logits (skyrl/tx/models/qwen3.py:172-185):
    ``(weights f32 [T, top_k], selected s32 [T, top_k])``."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    t = router_logits.shape[0]
    return _call(jax, TARGETS[6], (jax.ShapeDtypeStruct((t, top_k), jnp.float32),
                                   jax.ShapeDtypeStruct((t, top_k), jnp.int32)),
                 router_logits.astype(jnp.float32), norm_topk_prob=int(bool(norm_topk_prob)))


def moe_dispatch(tokens, indices, num_groups: int, *, repeat: int = 1, adapter_indices=None):
    """Stable sort of the (token, choice) pairs by group (``prepare_routing``, skyrl/tx/layers/util.py:66-87,
    for ``repeat == 1``): ``(sorted_tokens or None, group_sizes, sort_indices, unsort_indices, sorted_adapters
    or None)``.  ``tokens=None`` sorts the indices only."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    flat = indices.astype(jnp.int32).reshape(-1)
    pairs = flat.shape[0]
    empty = lambda dt, nd: jnp.zeros((0,) * nd, dt)
    tok = empty(jnp.bfloat16, 2) if tokens is None else tokens
    ad = empty(jnp.int32, 1) if adapter_indices is None else adapter_indices.astype(jnp.int32).reshape(-1)
    width = 0 if tokens is None else tokens.shape[1]
    ws = int(_native.load().mi355_w8a8_moe_dispatch_workspace_bytes(pairs, num_groups))
    if ws == 0:
        raise ValueError(f"{pairs} pairs over {num_groups} groups is outside the native path")
    st, gs, si, ui, sa, _ = _call(
        jax, TARGETS[7],
        (jax.ShapeDtypeStruct((pairs, width) if tokens is not None else (0, 0), jnp.bfloat16),
         jax.ShapeDtypeStruct((num_groups,), jnp.int32), jax.ShapeDtypeStruct((pairs,), jnp.int32),
         jax.ShapeDtypeStruct((pairs,), jnp.int32),
         jax.ShapeDtypeStruct((pairs,) if adapter_indices is not None else (0,), jnp.int32),
         jax.ShapeDtypeStruct((ws,), jnp.uint8)),
        tok, flat, ad, repeat=int(repeat))
    return (st if tokens is not None else None), gs, si, ui, (sa if adapter_indices is not None else None)


def moe_combine(expert_out, unsort_indices, weights):
    """``out[t] = sum_j expert_out[unsort[t * top_k + j]] * weights[t, j]`` (skyrl/tx/models/qwen3.py:203-210)."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    t = weights.shape[0]
    (out,) = _call(jax, TARGETS[8], (jax.ShapeDtypeStruct((t, expert_out.shape[1]), jnp.bfloat16),), expert_out,
                   unsort_indices.astype(jnp.int32), weights.astype(jnp.float32))
    return out


def grouped_backward(x, dy, packed_weights, w_scales, group_sizes, lora_a=None, lora_b=None, lora_scaling=None):
    """Cotangents of the grouped call as one XLA custom call: ``(dx, dA, dB, dscaling)`` (the LoRA entries
    ``None`` without LoRA) -- the backward rule a ``jax.custom_vjp`` around ``LoRAExpert.__call__``
    (skyrl/tx/layers/lora.py:394-444) binds."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    m, k = x.shape
    n = w_scales.shape[-1]
    n_groups = group_sizes.shape[0]
    n_weights = w_scales.reshape(-1, n).shape[0]
    empty = lambda dt, nd: jnp.zeros((0,) * nd, dt)
    a3 = empty(jnp.bfloat16, 3) if lora_a is None else lora_a
    b3 = empty(jnp.bfloat16, 3) if lora_b is None else lora_b
    rank = a3.shape[2] if lora_a is not None else 0
    s1 = (empty(jnp.float32, 1) if lora_a is None
          else jnp.broadcast_to(jnp.asarray(lora_scaling, jnp.float32), (n_groups,)))
    ws = int(_native.load().mi355_w8a8_grouped_bwd_workspace_bytes(m, k, n, n_groups, rank, n_groups // n_weights))
    if ws == 0:
        raise ValueError(f"geometry M={m}, K={k}, N={n}, groups={n_groups} is outside the native backward")
    dx, da, db, ds, _ = _call(
        jax, TARGETS[13],
        (jax.ShapeDtypeStruct((m, k), jnp.bfloat16), jax.ShapeDtypeStruct(a3.shape, jnp.bfloat16),
         jax.ShapeDtypeStruct(b3.shape, jnp.bfloat16), jax.ShapeDtypeStruct(s1.shape, jnp.float32),
         jax.ShapeDtypeStruct((ws,), jnp.uint8)),
        x, dy, packed_weights, w_scales.reshape(-1, n).astype(jnp.float32), a3, b3, s1, group_sizes.astype(jnp.int32))
    if lora_a is None:
        return dx, None, None, None
    return dx, da, db, ds


def qkv_split_norm_rope_backward(fused, q_norm_weight, k_norm_weight, positions, d_q, d_k, d_v, d_gate, *,
                                 rotary_dim: int, rope_theta: float, eps: float = 1e-6, want_weight_grads: bool = True):
    """Pull-back of ``qkv_split_norm_rope`` (skyrl/tx/kernels/qwen3_5_qkv_lora.py:391-425):
    ``(d_fused, d_q_norm_weight, d_k_norm_weight)``; the weight cotangents are ``None`` when not wanted."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    m, heads, head_dim = d_q.shape
    nw = head_dim if want_weight_grads else 0
    ws = int(_native.load().mi355_w8a8_qkv_bwd_workspace_bytes(m, head_dim)) if want_weight_grads else 0
    d_fused, dqw, dkw, _ = _call(
        jax, TARGETS[14],
        (jax.ShapeDtypeStruct(fused.shape, jnp.bfloat16), jax.ShapeDtypeStruct((nw,), jnp.float32),
         jax.ShapeDtypeStruct((nw,), jnp.float32), jax.ShapeDtypeStruct((ws,), jnp.uint8)),
        fused, q_norm_weight.astype(jnp.float32), k_norm_weight.astype(jnp.float32),
        positions.astype(jnp.int32).reshape(m), d_q, d_k, d_v, d_gate, rotary_dim=int(rotary_dim),
        rope_theta=float(rope_theta), rms_eps=float(eps))
    return (d_fused, dqw, dkw) if want_weight_grads else (d_fused, None, None)


def delta_rms_norm_backward(x, gamma, d_normalized, *, eps: float = 1e-6, want_gamma_grad: bool = True):
    """Pull-back of the decoder norm with multiplier ``gamma = 1 + weight``
    (skyrl/tx/kernels/qwen3_5_qkv_lora.py:97-116): ``(d_x, d_gamma or None)``."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    k = x.shape[-1]
    m = 1
    for d in x.shape[:-1]:
        m *= d
    ng = k if want_gamma_grad else 0
    ws = int(_native.load().mi355_w8a8_delta_rms_norm_bwd_workspace_bytes(m, k)) if want_gamma_grad else 0
    d_x, d_gamma, _ = _call(jax, TARGETS[15],
                            (jax.ShapeDtypeStruct(x.shape, jnp.bfloat16), jax.ShapeDtypeStruct((ng,), jnp.float32),
                             jax.ShapeDtypeStruct((ws,), jnp.uint8)),
                            x, gamma.astype(jnp.float32), d_normalized, eps=float(eps))
    return d_x, (d_gamma if want_gamma_grad else None)


def moe_route_backward(router_logits, selected, d_weights, norm_topk_prob: bool):
    """Cotangent of the router logits with the selection held fixed (skyrl/tx/models/qwen3.py:175-178)."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    (d_logits,) = _call(jax, TARGETS[16], (jax.ShapeDtypeStruct(router_logits.shape, jnp.float32),),
                        router_logits.astype(jnp.float32), selected.astype(jnp.int32), d_weights.astype(jnp.float32),
                        norm_topk_prob=int(bool(norm_topk_prob)))
    return d_logits


def moe_combine_backward(d_out, expert_out, sort_indices, weights):
    """Cotangents of the combine in its two operands (skyrl/tx/models/qwen3.py:205-207):
    ``(d_expert_out bf16 [T * top_k, H], d_weights f32 [T, top_k])``."""
    jax = _import_jax()
    register(jax)
    jnp = jax.numpy
    return _call(jax, TARGETS[17],
                 (jax.ShapeDtypeStruct(expert_out.shape, jnp.bfloat16), jax.ShapeDtypeStruct(weights.shape, jnp.float32)),
                 d_out, expert_out, sort_indices.astype(jnp.int32), weights.astype(jnp.float32))
