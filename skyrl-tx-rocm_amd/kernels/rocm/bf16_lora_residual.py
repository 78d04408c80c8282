"""``bf16_lora_residual`` with a W8A8 frozen kernel.

Same name, positional order and keywords as the reference's entry point
(skyrl/tx/kernels/rocm/bf16_lora_residual.py:507-522; call site ``Qwen3_5MLP._apply_down``,
skyrl/tx/models/qwen3_5.py:767-782); ``frozen_weight`` is a ``GroupQuantizedWeight`` instead of a bf16
matrix.  ``out = bf16(W8A8(x) + s * (x @ A) @ B + residual)``: the residual joins the float32
epilogue before the single cast.  Like the reference's custom VJP (:447-504) the call is
differentiable with respect to ``x``, LoRA A/B and the residual (and, here, the scaling); the
frozen kernel gets no gradient.  Tile keywords are validated and otherwise ignored.
"""

from __future__ import annotations

from .. import quantized_lora as ql
from . import w8a8_lora as w8

DEFAULT_BLOCK_M = 32
DEFAULT_BLOCK_N = 64
DEFAULT_BLOCK_K = 64
DEFAULT_ROW_SUPERBLOCK = 512


def bf16_lora_residual(x, frozen_weight, lora_a, lora_b, lora_scaling, residual, *, enabled: bool = False,
                       interpret: bool = False, block_m: int = DEFAULT_BLOCK_M, block_n: int = DEFAULT_BLOCK_N,
                       block_k: int = DEFAULT_BLOCK_K, row_superblock: int = DEFAULT_ROW_SUPERBLOCK,
                       pallas_input_vjp: bool = False, adapter_indices=None):
    w8._check_enabled(enabled, interpret, "LoRA residual")
    w8._validate_exact_bool("pallas_input_vjp", pallas_input_vjp)
    for name, value in (("block_m", block_m), ("block_n", block_n), ("block_k", block_k),
                        ("row_superblock", row_superblock)):
        if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
            raise ValueError(f"{name} must be a positive integer, got {value!r}")
    if not isinstance(frozen_weight, (ql.GroupQuantizedWeight, w8.PackedW8Weight)):
        raise TypeError("frozen_weight must be a GroupQuantizedWeight (quantize the bf16 kernel once with "
                        "quantize_frozen_weight(kernel, bits=8, group_size=K)); there is no bf16 GEMM path")
    return w8.w8a8_lora_residual(x, frozen_weight, lora_a, lora_b, lora_scaling, residual, enabled=True,
                                 adapter_indices=adapter_indices)


__all__ = ("bf16_lora_residual", "DEFAULT_BLOCK_M", "DEFAULT_BLOCK_N", "DEFAULT_BLOCK_K", "DEFAULT_ROW_SUPERBLOCK")
