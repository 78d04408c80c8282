"""Storage format and public entry points of the grouped-quantized LoRA linear.

Mirrors the interface of the reference's ``skyrl/tx/kernels/quantized_lora.py``
(``GroupQuantizedWeight`` :20-41, ``quantize_frozen_weight`` :128-171,
``dequantize_frozen_weight`` :180-196, ``quantized_frozen_linear`` :257-272,
``quantized_lora_linear`` :400-453) on torch tensors.  The forward functions run the
gfx950 HIP kernels: the per-token / per-channel geometry (``bits == 8``,
``group_size == K``, ``activation_bits == 8``) takes the tiled / streaming W8A8
kernels, every other geometry of the format (W4 codes, scales per K group, A4
activations, any group size) the group-scaled kernels of ``rocm/gq_linear.py``; under
autograd that path carries the reference's pullback on float32 library GEMMs.
The weight quantizer is an offline, one-time torch computation.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch


@dataclass(frozen=True)
class GroupQuantizedWeight:
    """K x N weight grouped along K with one scale per (group, output)."""

    codes: torch.Tensor
    scales: torch.Tensor
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
    if tuple(weight.scales.shape) != scale_shape:
        raise ValueError(f"scale shape {tuple(weight.scales.shape)} does not match expected {scale_shape}")
    if weight.codes.shape[1] <= 0:
        raise ValueError("quantized weight output dimension must be positive")
    want = torch.uint8 if weight.bits == 4 else torch.int8
    if weight.codes.dtype != want:
        raise TypeError(f"W{weight.bits} codes must have dtype {want}, got {weight.codes.dtype}")
    if not weight.scales.dtype.is_floating_point:
        raise TypeError(f"quantized weight scales must be floating point, got {weight.scales.dtype}")


def pack_signed_int4(values: torch.Tensor) -> torch.Tensor:
    if values.ndim < 1 or values.shape[0] == 0 or values.shape[0] % 2:
        raise ValueError("signed INT4 packing requires an even, nonempty axis zero")
    if values.dtype.is_floating_point or values.dtype == torch.bool:
        raise TypeError(f"signed INT4 values must be integral, got {values.dtype}")
    low = (values[0::2].to(torch.int16) & 0xF).to(torch.uint8)
    high = (values[1::2].to(torch.int16) & 0xF).to(torch.uint8)
    return low | (high << 4)


def unpack_signed_int4(packed: torch.Tensor) -> torch.Tensor:
    if packed.ndim < 1 or packed.shape[0] == 0:
        raise ValueError("signed INT4 input must have a nonempty axis zero")
    if packed.dtype != torch.uint8:
        raise TypeError(f"packed signed INT4 values must be uint8, got {packed.dtype}")
    low = (packed & 0xF).to(torch.int16)
    high = (packed >> 4).to(torch.int16)
    low = torch.where(low >= 8, low - 16, low).to(torch.int8)
    high = torch.where(high >= 8, high - 16, high).to(torch.int8)
    return torch.stack((low, high), dim=1).reshape((packed.shape[0] * 2, *packed.shape[1:]))


def quantize_frozen_weight(weight: torch.Tensor, *, bits: int = 8, group_size: int = 64,
                           scale_dtype: torch.dtype = torch.bfloat16) -> GroupQuantizedWeight:
    """Symmetric per-(group, output) quantizer (offline, once per weight)."""
    _validate_bits(bits)
    _validate_group_size(group_size)
    if weight.ndim != 2:
        raise ValueError(f"weight must have shape [K, N], got {tuple(weight.shape)}")
    if weight.shape[0] <= 0 or weight.shape[1] <= 0:
        raise ValueError(f"weight dimensions must be positive, got {tuple(weight.shape)}")
    if not weight.dtype.is_floating_point:
        raise TypeError(f"weight must be floating point, got {weight.dtype}")
    if not scale_dtype.is_floating_point:
        raise TypeError(f"scale_dtype must be floating point, got {scale_dtype}")
    k, n = weight.shape
    k_pad = ((k + group_size - 1) // group_size) * group_size
    padded = torch.zeros((k_pad, n), dtype=torch.float32, device=weight.device)
    padded[:k] = weight.to(torch.float32)
    grouped = padded.reshape(-1, group_size, n)
    qmax = (1 << (bits - 1)) - 1
    amax = grouped.abs().amax(dim=1)
    scales = torch.where(amax > 0, amax / qmax, torch.ones_like(amax))
    q = torch.clamp(torch.round(grouped / scales[:, None, :]), -qmax, qmax).to(torch.int8)
    q = q.reshape(k_pad, n)
    codes = q if bits == 8 else pack_signed_int4(q)
    return GroupQuantizedWeight(codes=codes, scales=scales.to(scale_dtype), original_in_features=k,
                                padded_in_features=k_pad, bits=bits, group_size=group_size)


def dequantize_frozen_weight(weight: GroupQuantizedWeight, *, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    validate_quantized_weight(weight)
    if not dtype.is_floating_point:
        raise TypeError(f"dequantized weight dtype must be floating point, got {dtype}")
    codes = weight.codes if weight.bits == 8 else unpack_signed_int4(weight.codes)
    codes = codes[: weight.padded_in_features]
    n = codes.shape[1]
    grouped = codes.reshape(-1, weight.group_size, n).to(torch.float32)
    deq = grouped * weight.scales.to(torch.float32)[:, None, :]
    return deq.reshape(weight.padded_in_features, n)[: weight.original_in_features].to(dtype)


def _is_per_channel_w8a8(weight: GroupQuantizedWeight, activation_bits: int) -> bool:
    """True for the geometry of the fast W8A8 kernels; validates the arguments either way."""
    _validate_bits(activation_bits)
    validate_quantized_weight(weight)
    # (K not a multiple of 8 goes the group-scaled way, embedded as one group of the next multiple of 32)
    return (weight.bits == 8 and activation_bits == 8 and weight.group_size == weight.padded_in_features
            and weight.padded_in_features == weight.original_in_features and weight.original_in_features % 8 == 0)


def _group_scaled_input_pullback(dy: torch.Tensor, weight: GroupQuantizedWeight) -> torch.Tensor:
    """``dy @ (codes * scales).T`` in float32, a slab of K groups at a time (quantized_lora.py:355-378: the
    dequantized K x N matrix is never held as a whole), cut to the original K."""
    codes = weight.codes if weight.bits == 8 else unpack_signed_int4(weight.codes)
    codes = codes[: weight.padded_in_features]
    n = codes.shape[1]
    g = weight.group_size
    n_groups = weight.padded_in_features // g
    scales = weight.scales.to(torch.float32)
    per_slab = max(1, (1 << 24) // max(1, g * n))  # about 64 MiB of float32 weight at a time
    parts = []
    for g0 in range(0, n_groups, per_slab):
        g1 = min(n_groups, g0 + per_slab)
        slab = codes[g0 * g: g1 * g].reshape(g1 - g0, g, n).to(torch.float32) * scales[g0:g1, None, :]
        parts.append(dy @ slab.reshape((g1 - g0) * g, n).T)
    return torch.cat(parts, dim=1)[:, : weight.original_in_features]


class _GroupScaledLoraFunction(torch.autograd.Function):
    """The group-scaled forward with the reference's pullback (quantized_lora.py:337-394): straight through
    the quantizers, ``dx = dy @ deq(W).T + r @ A.T`` with ``r = (dy @ B.T) * s``, ``dA = x.T @ r``,
    ``dB = ((x @ A).T @ dy) * s``, ``ds = sum(dy * ((x @ A) @ B))``, all in float32 on the library GEMMs and
    cast once.  The frozen weight gets no gradient."""

    @staticmethod
    def forward(ctx, x, lora_a, lora_b, scaling, weight, activation_bits):
        from .rocm import gq_linear

        ctx.save_for_backward(x, lora_a, lora_b, scaling)
        ctx.weight = weight
        return gq_linear.forward(x, weight, lora_a, lora_b, scaling, activation_bits=activation_bits)

    @staticmethod
    def backward(ctx, dy):
        x, lora_a, lora_b, scaling = ctx.saved_tensors
        weight = ctx.weight
        xf = x.reshape(-1, x.shape[-1]).to(torch.float32)
        dyf = dy.reshape(-1, dy.shape[-1]).to(torch.float32)
        a, b = lora_a.to(torch.float32), lora_b.to(torch.float32)
        s = scaling.to(device=dyf.device, dtype=torch.float32)
        z = xf @ a
        r = (dyf @ b.T) * s
        dx = da = db = ds = None
        if ctx.needs_input_grad[0]:
            dx = (_group_scaled_input_pullback(dyf, weight) + r @ a.T).reshape(x.shape).to(x.dtype)
        if ctx.needs_input_grad[1]:
            da = (xf.T @ r).to(lora_a.dtype)
        if ctx.needs_input_grad[2]:
            db = ((z.T @ dyf) * s).to(lora_b.dtype)
        if ctx.needs_input_grad[3]:
            ds = (dyf * (z @ b)).sum().reshape(scaling.shape).to(scaling.dtype)
        return dx, da, db, ds, None, None


def quantized_frozen_linear(x: torch.Tensor, weight: GroupQuantizedWeight, *, activation_bits: int = 8):
    from .rocm import gq_linear, w8a8_lora

    per_channel = _is_per_channel_w8a8(weight, activation_bits)
    if not x.dtype.is_floating_point:
        raise TypeError(f"activations must be floating point, got {x.dtype}")
    if per_channel:
        return w8a8_lora.w8a8_frozen_linear(x, weight, enabled=True)
    return gq_linear.forward(x, weight, activation_bits=activation_bits)


def quantized_lora_linear(x: torch.Tensor, weight: GroupQuantizedWeight, lora_a: torch.Tensor,
                          lora_b: torch.Tensor, lora_scaling, *, activation_bits: int = 8) -> torch.Tensor:
    """Frozen W8A8 linear plus LoRA: bf16(base_f32 + ((x @ A) @ B) * s), one cast."""
    from .rocm import gq_linear, w8a8_lora

    per_channel = _is_per_channel_w8a8(weight, activation_bits)
    if x.ndim < 1:
        raise ValueError(f"activations must have at least one dimension, got {tuple(x.shape)}")
    if not x.dtype.is_floating_point:
        raise TypeError(f"activations must be floating point, got {x.dtype}")
    if lora_a.ndim != 2 or lora_b.ndim != 2:
        raise ValueError("lora_a and lora_b must both be rank-two")
    if not lora_a.dtype.is_floating_point or not lora_b.dtype.is_floating_point:
        raise TypeError(f"LoRA parameters must be floating point, got {lora_a.dtype} and {lora_b.dtype}")
    if tuple(lora_a.shape) != (weight.original_in_features, lora_b.shape[0]):
        raise ValueError(
            f"incompatible LoRA shapes: A={tuple(lora_a.shape)}, B={tuple(lora_b.shape)}, "
            f"weight K={weight.original_in_features}")
    if lora_b.shape[1] != weight.codes.shape[-1]:
        raise ValueError(f"LoRA output N={lora_b.shape[1]} does not match weight N={weight.codes.shape[-1]}")
    scaling = torch.as_tensor(lora_scaling, dtype=torch.float32)
    if scaling.ndim != 0:
        raise ValueError(f"lora_scaling must be scalar, got {tuple(scaling.shape)}")
    if per_channel:
        return w8a8_lora.w8a8_lora_linear(x, weight, lora_a, lora_b, scaling, enabled=True)
    if torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad
                                       for t in (x, lora_a, lora_b, lora_scaling)):
        s_arg = lora_scaling if isinstance(lora_scaling, torch.Tensor) and lora_scaling.requires_grad else scaling
        return _GroupScaledLoraFunction.apply(x, lora_a, lora_b, s_arg, weight, activation_bits)
    return gq_linear.forward(x, weight, lora_a, lora_b, scaling, activation_bits=activation_bits)
