"""Group-scaled quantized linear on the native kernels: W4 or W8 codes with one scale per
(K group, output), A4 or A8 activations quantized per (row, K group) -- the general form of
``quantized_frozen_linear`` / ``quantized_lora_linear`` (skyrl/tx/kernels/quantized_lora.py:215-304).

The per-token / per-channel W8A8 case (``group_size == K``) has its own, much faster kernels in
``w8a8_lora``; everything else the storage format allows (``bits`` 4, ``group_size`` < K,
``activation_bits`` 4) comes here.  The packed weight keeps 4-bit codes at half a byte per weight.
"""

from __future__ import annotations

import ctypes
import threading
import weakref
from dataclasses import dataclass

import torch

from ... import _native
from .. import quantized_lora as ql
from .w8a8_lora import MAX_LORA_RANK, _require_cuda, _stream_ptr, _version_of


@dataclass(frozen=True)
class PackedGroupWeight:
    """A ``GroupQuantizedWeight`` re-laid into matrix-core fragments (``mi355_w8a8_gq_pack_weight_v1``)."""

    packed: torch.Tensor       # uint8
    scales: torch.Tensor       # f32 [K_pad / group_size, N]
    in_features: int
    padded_in_features: int
    out_features: int
    bits: int
    group_size: int
    # The reference's own group size and padded K where they differ from the packed ones: a group size that is
    # not a multiple of 32 is embedded, every group followed by zero codes up to the next multiple of 32 (and x
    # by zeros at the same places), which changes no maximum, no code of a real element and no integer sum.
    source_group_size: int = 0
    source_padded_in_features: int = 0


_pack_cache: dict = {}
_pack_lock = threading.Lock()


def prepare_group_weight(weight) -> PackedGroupWeight:
    """Pack once per weight (cached on the codes tensor): the load-time re-layout."""
    if isinstance(weight, PackedGroupWeight):
        return weight
    ql.validate_quantized_weight(weight)
    codes = weight.codes
    _require_cuda(codes, "weight codes")
    key = (codes.data_ptr(), weight.scales.data_ptr(), weight.padded_in_features, codes.shape[1], weight.bits,
           weight.group_size, _version_of(codes), _version_of(weight.scales))
    with _pack_lock:
        hit = _pack_cache.get(key)
        if hit is not None and hit[0]() is codes:
            return hit[1]
    want = torch.uint8 if weight.bits == 4 else torch.int8
    if codes.dtype != want:
        raise TypeError(f"W{weight.bits} codes must have dtype {want}, got {codes.dtype}")
    k_pad, n = weight.padded_in_features, codes.shape[1]
    group, src_group, src_k_pad = weight.group_size, 0, 0
    if group % 32:
        # embed: [G, group, N] -> [G, group32, N] with zero codes behind every group
        src_group, src_k_pad = group, k_pad
        group32 = (group + 31) // 32 * 32
        n_groups = k_pad // group
        plain = (codes if weight.bits == 8 else ql.unpack_signed_int4(codes))[:k_pad]
        wide = torch.zeros((n_groups, group32, n), dtype=torch.int8, device=codes.device)
        wide[:, :group] = plain.reshape(n_groups, group, n)
        wide = wide.reshape(n_groups * group32, n)
        codes = wide if weight.bits == 8 else ql.pack_signed_int4(wide)
        group, k_pad = group32, n_groups * group32
    lib = _native.load()
    nbytes = int(lib.mi355_w8a8_gq_packed_weight_bytes(k_pad, n, weight.bits))
    if nbytes == 0:
        raise ValueError(f"geometry K_pad={k_pad}, N={n}, bits={weight.bits} is outside the native path")
    src = codes.contiguous()
    packed = torch.empty(nbytes, dtype=torch.uint8, device=codes.device)
    with torch.cuda.device(codes.device):
        status = lib.mi355_w8a8_gq_pack_weight_v1(src.data_ptr(), packed.data_ptr(), k_pad, n, weight.bits,
                                                  _stream_ptr(codes.device))
    _native.check("mi355_w8a8_gq_pack_weight_v1", status)
    out = PackedGroupWeight(packed, weight.scales.to(torch.float32).contiguous(), weight.original_in_features, k_pad,
                            n, weight.bits, group, src_group, src_k_pad)
    with _pack_lock:
        if len(_pack_cache) > 4096:
            _pack_cache.clear()
        _pack_cache[key] = (weakref.ref(weight.codes), out)
    return out


def forward(x: torch.Tensor, weight, lora_a=None, lora_b=None, lora_scaling=None, *, activation_bits: int = 8,
            adapter_indices: torch.Tensor | None = None, return_aux: bool = False, flags: int = 0):
    """bf16(base + s[idx] * ((x @ A[idx]) @ B[idx])) with the grouped-scale base of
    quantized_lora.py:215-254.  ``lora_a`` / ``lora_b`` are [K, r] / [r, N] with a scalar scaling, or
    stacked [n, K, r] / [n, r, N] with ``lora_scaling`` [n] and one adapter index per row.
    ``flags``: 0, or ``_native.FLAG_GQ_DIRECT`` for the kernel without LDS staging (same bits)."""
    if activation_bits not in (4, 8):
        raise ValueError(f"bits must be 4 or 8, got {activation_bits}")
    if x.dtype != torch.bfloat16:
        raise TypeError(f"x must be BF16, got {x.dtype}")
    _require_cuda(x, "x")
    pw = prepare_group_weight(weight)
    k, n = pw.in_features, pw.out_features
    if x.ndim < 1 or x.shape[-1] != k or x.numel() == 0:
        raise ValueError(f"activation K={x.shape[-1] if x.ndim else None} does not match weight K={k}")
    dev = x.device
    flat = x.reshape(-1, k).contiguous()
    m = flat.shape[0]

    def embed(t, axis):  # the K axis of x (or of LoRA A) with zeros behind every source group
        src_g, dst_g, n_groups = pw.source_group_size, pw.group_size, pw.padded_in_features // pw.group_size
        shape = list(t.shape)
        padded = torch.zeros(shape[:axis] + [pw.source_padded_in_features] + shape[axis + 1:], dtype=t.dtype, device=dev)
        padded.narrow(axis, 0, k).copy_(t)
        wide = torch.zeros(shape[:axis] + [n_groups, dst_g] + shape[axis + 1:], dtype=t.dtype, device=dev)
        wide.narrow(axis + 1, 0, src_g).copy_(padded.reshape(shape[:axis] + [n_groups, src_g] + shape[axis + 1:]))
        return wide.reshape(shape[:axis] + [n_groups * dst_g] + shape[axis + 1:])

    embedded = pw.source_group_size != 0
    if embedded:
        flat = embed(flat, 1)
    a3 = b3 = s1 = idx = None
    n_ad = r = 0
    if lora_a is not None:
        if lora_a.dtype != torch.bfloat16 or lora_b.dtype != torch.bfloat16:
            raise TypeError("LoRA A and B must both be BF16")
        a3 = lora_a if lora_a.ndim == 3 else lora_a[None]
        b3 = lora_b if lora_b.ndim == 3 else lora_b[None]
        n_ad, r = a3.shape[0], a3.shape[2]
        if a3.ndim != 3 or b3.ndim != 3 or tuple(a3.shape) != (n_ad, k, r) or tuple(b3.shape) != (n_ad, r, n):
            raise ValueError(f"incompatible LoRA shapes: A={tuple(lora_a.shape)}, B={tuple(lora_b.shape)}, weight "
                             f"K={k}, N={n}")
        if r < 1 or r > MAX_LORA_RANK:
            raise ValueError(f"LoRA rank must be in [1, {MAX_LORA_RANK}], got {r}")
        a3, b3 = (embed(a3, 1) if embedded else a3).contiguous(), b3.contiguous()
        s1 = torch.as_tensor(lora_scaling, dtype=torch.float32, device=dev).reshape(-1)
        s1 = (s1.expand(n_ad) if s1.numel() == 1 else s1).contiguous()
        if s1.numel() != n_ad:
            raise ValueError(f"lora_scaling must be a scalar or have {n_ad} entries")
        if adapter_indices is not None:
            idx = adapter_indices.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
            if idx.numel() != m:
                raise ValueError(f"adapter_indices must hold one entry per row ({m}), got {idx.numel()}")
    elif adapter_indices is not None:
        raise ValueError("adapter_indices given without LoRA parameters")
    lib = _native.load()
    ws_bytes = int(lib.mi355_w8a8_gq_workspace_bytes(m, pw.padded_in_features, pw.group_size, n_ad, r))
    if ws_bytes == 0:
        raise ValueError(f"geometry M={m}, K_pad={pw.padded_in_features}, group={pw.group_size}, rank={r} is outside "
                         "the native path")
    out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    aux = {}
    if return_aux:
        groups = pw.padded_in_features // pw.group_size
        aux["x_codes"] = torch.empty((m, pw.padded_in_features), dtype=torch.int8, device=dev)
        aux["x_scales"] = torch.empty((m, groups), dtype=torch.float32, device=dev)
        aux["base"] = torch.empty((m, n), dtype=torch.float32, device=dev)
    p = _native.GqProblem()
    p.struct_size = ctypes.sizeof(_native.GqProblem)
    p.flags = int(flags)
    p.m, p.k, p.k_pad, p.n = m, (pw.padded_in_features if embedded else k), pw.padded_in_features, n
    p.group_size, p.weight_bits, p.activation_bits = pw.group_size, pw.bits, activation_bits
    p.n_adapters, p.rank = n_ad, r
    p.x = flat.data_ptr()
    p.w_packed = pw.packed.data_ptr()
    p.w_scales = pw.scales.data_ptr()
    p.lora_a = a3.data_ptr() if n_ad else None
    p.lora_b = b3.data_ptr() if n_ad else None
    p.lora_scaling = s1.data_ptr() if n_ad else None
    p.adapter_indices = idx.data_ptr() if idx is not None else None
    p.out = out.data_ptr()
    p.workspace = ws.data_ptr()
    p.workspace_bytes = ws_bytes
    p.aux_x_codes = aux["x_codes"].data_ptr() if return_aux else None
    p.aux_x_scales = aux["x_scales"].data_ptr() if return_aux else None
    p.aux_base = aux["base"].data_ptr() if return_aux else None
    with torch.cuda.device(dev):
        status = lib.mi355_w8a8_gq_linear_v1(ctypes.byref(p), _stream_ptr(dev))
    _native.check("mi355_w8a8_gq_linear_v1", status)
    result = out.reshape(*x.shape[:-1], n)
    if return_aux and embedded:  # the codes in the reference's own layout, without the zeros of the embedding
        n_groups = pw.padded_in_features // pw.group_size
        aux["x_codes"] = aux["x_codes"].reshape(m, n_groups, pw.group_size)[:, :, :pw.source_group_size].reshape(
            m, pw.source_padded_in_features).contiguous()
    return (result, aux) if return_aux else result


__all__ = ("PackedGroupWeight", "prepare_group_weight", "forward")
