"""``bf16_rms_gate_up_lora_swiglu_contiguous`` with a W8A8 frozen kernel.

Same name, positional order and keywords as the reference's entry point
(skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:698-712), so a call site such as
``Qwen3_5MLP._bf16_rms_gate_up_lora_swiglu_contiguous`` (skyrl/tx/models/qwen3_5.py:746-759) keeps its
shape; ``frozen_weight`` is a ``GroupQuantizedWeight`` (int8 codes, one scale per output channel,
columns interleaved gate0, up0, gate1, up1, ...) instead of a bf16 matrix.  RMSNorm with
``1 + rms_delta``, the W8A8 gate/up projection, LoRA and SwiGLU run as one native forward call.
Tile keywords are validated as exact integers and otherwise ignored.  Under autograd the call has
the reference's derivative rule (:643-689): cotangents for ``x``, ``lora_a``, ``lora_b``; none for
``rms_delta`` and the frozen kernel.
"""

from __future__ import annotations

import torch

from .. import quantized_lora as ql
from . import w8a8_lora as w8

RMS_NORM_EPSILON = 1e-6
DEFAULT_BLOCK_M = 16
DEFAULT_BLOCK_PHYSICAL_N = 64
DEFAULT_BLOCK_K = 64


def _check_tile(name: str, value) -> None:
    if isinstance(value, bool) or not isinstance(value, int) or value <= 0:
        raise ValueError(f"{name} must be a positive integer, got {value!r}")


def bf16_rms_gate_up_lora_swiglu_contiguous(x, rms_delta, frozen_weight, lora_a, lora_b, lora_scaling, *,
                                            enabled: bool = False, eps: float = RMS_NORM_EPSILON,
                                            interpret: bool = False, block_m: int = DEFAULT_BLOCK_M,
                                            block_physical_n: int = DEFAULT_BLOCK_PHYSICAL_N,
                                            block_k: int = DEFAULT_BLOCK_K, adapter_indices=None):
    w8._check_enabled(enabled, interpret, "RMSNorm gate/up SwiGLU")
    if not isinstance(eps, float) or not eps > 0.0:
        raise ValueError(f"eps must be a positive float, got {eps!r}")
    for name, value in (("block_m", block_m), ("block_physical_n", block_physical_n), ("block_k", block_k)):
        _check_tile(name, value)
    if not isinstance(frozen_weight, (ql.GroupQuantizedWeight, w8.PackedW8Weight)):
        raise TypeError("frozen_weight must be a GroupQuantizedWeight (quantize the bf16 kernel once with "
                        "quantize_frozen_weight(kernel, bits=8, group_size=K)); there is no bf16 GEMM path")
    return w8.w8a8_rms_gate_up_lora_swiglu(x, rms_delta, frozen_weight, lora_a, lora_b, lora_scaling,
                                           enabled=True, eps=eps, rms_is_delta=True,
                                           adapter_indices=adapter_indices)


__all__ = ("bf16_rms_gate_up_lora_swiglu_contiguous", "RMS_NORM_EPSILON", "DEFAULT_BLOCK_M",
           "DEFAULT_BLOCK_PHYSICAL_N", "DEFAULT_BLOCK_K")
