"""``bounded_frozen_lora_linear`` with a W8A8 frozen kernel.

The reference's module (skyrl/tx/kernels/bounded_lora.py) is a CPU/JAX statement of one stage,

    Y = X W + scaling * (X A) B  (+ residual),

evaluated over row tiles of ``token_tile_size`` so that its temporaries stay bounded, for "a future
bounded ROCm HIP/FFI operation" (:1-16).  Here that operation exists: same name, positional order and
keywords (:245-255), the same argument checks (:31-108: exact-int tile size in [1, 2048], rank-two
single-adapter factors of rank 8, a floating scalar scaling, residual of the output's shape and dtype),
``frozen_weight`` a ``GroupQuantizedWeight`` instead of a dense matrix.  Rows are independent in the
forward, so the result does not depend on ``token_tile_size`` (what the reference's test pins,
tests/tx/kernels/test_bounded_lora.py:23-43); the native call's temporaries are bounded by its workspace,
which holds codes and tables of the rows of one call, so a caller that wants the reference's memory
bound passes its rows in pieces of that size -- the results are the same bits.  Differentiable in x, A,
B (and the residual, whose cotangent is the output's), like the reference's custom VJP (:149-243); the
frozen kernel and the scaling of the reference receive none there, the scaling does here.
"""

from __future__ import annotations

import math

import torch

from . import quantized_lora as ql
from .rocm import w8a8_lora as w8

LORA_RANK = 8
MAX_TOKEN_TILE_SIZE = 2048


def _validate_token_tile_size(token_tile_size: int) -> None:
    if isinstance(token_tile_size, bool) or not isinstance(token_tile_size, int):
        raise TypeError("token_tile_size must be an integer")
    if not 1 <= token_tile_size <= MAX_TOKEN_TILE_SIZE:
        raise ValueError(f"token_tile_size must be in [1, {MAX_TOKEN_TILE_SIZE}], got {token_tile_size}")


def bounded_frozen_lora_linear(x, frozen_weight, lora_a, lora_b, lora_scaling, *, residual=None,
                               token_tile_size: int = 512):
    _validate_token_tile_size(token_tile_size)
    if x.ndim < 1 or math.prod(x.shape[:-1]) <= 0:
        raise ValueError(f"x must have a nonempty row domain and final K axis, got {tuple(x.shape)}")
    if not isinstance(frozen_weight, (ql.GroupQuantizedWeight, w8.PackedW8Weight)):
        raise TypeError("frozen_weight must be a GroupQuantizedWeight (quantize the kernel once with "
                        "quantize_frozen_weight(kernel, bits=8, group_size=K)); there is no dense GEMM path")
    if lora_a.ndim != 2 or lora_b.ndim != 2:
        raise ValueError("single-adapter lora_a and lora_b must both be rank-two")
    if x.dtype != torch.bfloat16:
        raise TypeError(f"x dtype must be BF16, got {x.dtype}")
    for name, value in (("lora_a", lora_a), ("lora_b", lora_b)):
        if value.dtype != x.dtype:
            raise TypeError(f"{name} dtype {value.dtype} must match x dtype {x.dtype}")
    if isinstance(frozen_weight, w8.PackedW8Weight):
        in_features, out_features = frozen_weight.in_features, frozen_weight.out_features
    else:
        in_features, out_features = frozen_weight.original_in_features, frozen_weight.codes.shape[1]
    if x.shape[-1] != in_features:
        raise ValueError(f"x K={x.shape[-1]} does not match frozen_weight K={in_features}")
    if tuple(lora_a.shape) != (in_features, LORA_RANK):
        raise ValueError(f"lora_a must have shape ({in_features}, {LORA_RANK}), got {tuple(lora_a.shape)}")
    if tuple(lora_b.shape) != (LORA_RANK, out_features):
        raise ValueError(f"lora_b must have shape ({LORA_RANK}, {out_features}), got {tuple(lora_b.shape)}")
    if isinstance(lora_scaling, torch.Tensor):
        if lora_scaling.ndim != 0 or not lora_scaling.dtype.is_floating_point:
            raise TypeError(f"lora_scaling must be a floating scalar, got shape={tuple(lora_scaling.shape)}, "
                            f"dtype={lora_scaling.dtype}")
    elif isinstance(lora_scaling, bool) or not isinstance(lora_scaling, (int, float)):
        raise TypeError(f"lora_scaling must be a floating scalar, got {lora_scaling!r}")
    expected = (*x.shape[:-1], out_features)
    if residual is not None:
        if tuple(residual.shape) != expected:
            raise ValueError(f"residual shape {tuple(residual.shape)} must match output shape {expected}")
        if residual.dtype != x.dtype:
            raise TypeError(f"residual dtype {residual.dtype} must match x dtype {x.dtype}")
    return w8.lora_linear(x, frozen_weight, lora_a, lora_b, lora_scaling, residual=residual)


__all__ = ("bounded_frozen_lora_linear", "LORA_RANK", "MAX_TOKEN_TILE_SIZE")
