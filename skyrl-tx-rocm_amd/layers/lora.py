"""LoRA layer modules of the reference on W8A8 frozen weights.

Mirrors the call surface of ``skyrl/tx/layers/lora.py``: ``LoRALinear.__call__(x,
adapter_indices=None)`` (:226-268), ``FusedLoRALinear.__call__ -> tuple`` with
``fuse``/``split`` (:271-351), ``LoRAExpert.__call__(x, group_sizes,
adapter_indices_sorted=None, *, group_offset=None)`` (:354-444) and
``init_lora_adapter`` (:447-501).  The frozen kernel is a ``GroupQuantizedWeight`` with one
group over K (int8 codes, one float32 scale per output channel) instead of a dense matrix;
the forward runs on the HIP kernels.  Parameters are plain torch tensors on the GPU: the
reference's flax/NNX containers, sharding annotations and RNG plumbing are not part of the path.
"""

from __future__ import annotations

import math

import torch

from ..kernels import quantized_lora as ql
from ..kernels.rocm import w8a8_lora as w8


class LoRAMixin:
    """Multi-adapter LoRA state and ``apply`` (skyrl/tx/layers/lora.py:12-157)."""

    def init_lora(self, *, max_lora_adapters: int, max_lora_rank: int, shape_A, shape_B, device) -> None:
        self.max_lora_adapters = int(max_lora_adapters)
        self.max_lora_rank = int(max_lora_rank)
        if self.max_lora_adapters == 0:
            self.lora_scaling = self.lora_ranks = self.lora_A = self.lora_B = None
            return
        self.lora_scaling = torch.ones(self.max_lora_adapters, dtype=torch.float32, device=device)
        self.lora_ranks = torch.full((self.max_lora_adapters,), self.max_lora_rank, dtype=torch.int32,
                                     device=device)
        # zeros until init_lora_adapter() is called (lora.py:48-63)
        self.lora_A = torch.zeros(shape_A, dtype=torch.bfloat16, device=device)
        self.lora_B = torch.zeros(shape_B, dtype=torch.bfloat16, device=device)

    def _lora_active(self, adapter_indices) -> bool:
        if self.max_lora_adapters == 0 or adapter_indices is None:
            return False
        if self.lora_A is None or self.lora_B is None or self.lora_scaling is None:
            raise RuntimeError("LoRA parameters are not initialized. `init_lora` must be called.")
        return True


class LoRALinear(LoRAMixin):
    """Linear layer with multi-adapter LoRA on a W8A8 frozen kernel.

    ``adapter_indices`` holds one adapter per example (leading dimension of ``x``) and is repeated
    per token, as in ``LoRAMixin.apply_lora`` (lora.py:118-157); rows are sorted and un-sorted
    inside the native call.  ``out = bf16(W8A8(x) + s[idx] * (x @ A[idx]) @ B[idx])`` with one
    cast (skyrl/tx/kernels/quantized_lora.py:298-299).  When ``x`` or a LoRA tensor requires a
    gradient the call is differentiable through the native backward (the reference's custom VJP,
    quantized_lora.py:337-394).
    """

    def __init__(self, in_features: int, out_features: int, *, weight: ql.GroupQuantizedWeight | None = None,
                 max_lora_adapters: int = 0, max_lora_rank: int = 8, use_bias: bool = False, device="cuda:0",
                 **_unused_reference_keywords):
        # sharding, dtype, param_dtype, kernel_init, bias_init and rngs of the reference are accepted
        # and ignored: they configure flax parameters, not the computation.
        self.in_features, self.out_features = int(in_features), int(out_features)
        self.device = torch.device(device)
        self.bias = torch.zeros(out_features, dtype=torch.bfloat16, device=self.device) if use_bias else None
        self.weight = None
        if weight is not None:
            self.load_quantized(weight)
        self.init_lora(max_lora_adapters=max_lora_adapters, max_lora_rank=max_lora_rank,
                       shape_A=(max_lora_adapters, in_features, max_lora_rank),
                       shape_B=(max_lora_adapters, max_lora_rank, out_features), device=self.device)

    def load_quantized(self, weight: ql.GroupQuantizedWeight) -> None:
        ql.validate_quantized_weight(weight)
        if weight.original_in_features != self.in_features or weight.codes.shape[-1] != self.out_features:
            raise ValueError(f"quantized weight is [{weight.original_in_features}, {weight.codes.shape[-1]}], "
                             f"layer is [{self.in_features}, {self.out_features}]")
        self.weight = weight

    def load_dense(self, kernel: torch.Tensor) -> None:
        """Quantize a dense [in, out] kernel per output channel (one group over K)."""
        self.load_quantized(ql.quantize_frozen_weight(kernel.to(self.device), bits=8, group_size=self.in_features,
                                                      scale_dtype=torch.float32))

    def __call__(self, x: torch.Tensor, adapter_indices: torch.Tensor | None = None) -> torch.Tensor:
        if self.weight is None:
            raise RuntimeError("the frozen kernel is not loaded: call load_quantized() or load_dense()")
        if self._lora_active(adapter_indices):
            if adapter_indices.shape[0] != x.shape[0]:
                raise ValueError("adapter_indices must hold one entry per example (leading axis of x)")
            out = w8.lora_linear(x, self.weight, self.lora_A, self.lora_B, self.lora_scaling,
                                 adapter_indices=adapter_indices)
        else:
            out = w8.lora_linear(x, self.weight)
        # The bias is a second bf16 addition after the fused call's single cast.  The reference's layer
        # rounds twice as well (nnx.Linear adds the bias to the base output, apply_lora then adds the
        # low-rank term, layers/lora.py:262-268), in the other order; Qwen3 projections carry no bias.
        return out if self.bias is None else out + self.bias


class FusedLoRALinear(LoRALinear):
    """LoRALinear whose output interleaves several component projections (lora.py:271-351)."""

    def __init__(self, in_features: int, out_features: int, *, components: tuple[str, ...],
                 group_sizes: tuple[int, ...], **kwargs):
        super().__init__(in_features, out_features, **kwargs)
        if len(components) != len(group_sizes):
            raise ValueError("one group size per component")
        self.components = tuple(components)
        self.group_sizes = tuple(int(g) for g in group_sizes)

    def __call__(self, x: torch.Tensor, adapter_indices: torch.Tensor | None = None) -> tuple[torch.Tensor, ...]:
        return self.split(super().__call__(x, adapter_indices), self.group_sizes)

    def load_components(self, kernels) -> None:
        """Checkpoint step for a fused projection (skyrl/tx/utils/models.py:159-191,330-339): the
        component kernels ``[in, out_i]`` are interleaved group by group on the host, then quantized
        per output channel and packed once."""
        kernels = list(kernels)
        if len(kernels) != len(self.components):
            raise ValueError(f"expected one kernel per component {self.components}, got {len(kernels)}")
        self.load_dense(self.fuse(*[k.to(torch.float32) for k in kernels], group_sizes=self.group_sizes))

    def load_split_adapter(self, adapter_index: int, lora_a_parts, lora_b_parts) -> None:
        """Load an adapter trained on the split projections: the branches must share one ``lora_A``
        (models.py:149-156); their ``lora_B`` are interleaved like the kernels."""
        a0 = lora_a_parts[0]
        if not all(torch.allclose(a0.float(), part.float()) for part in lora_a_parts[1:]):
            raise RuntimeError("Cannot load split LoRA adapter into fused projection because the source "
                               "branches do not share the same lora_A matrix.")
        if not 0 <= adapter_index < self.max_lora_adapters:
            raise ValueError(f"adapter_index {adapter_index} outside [0, {self.max_lora_adapters})")
        fused_b = self.fuse(*lora_b_parts, group_sizes=self.group_sizes)
        with torch.no_grad():
            self.lora_A[adapter_index] = a0.to(device=self.lora_A.device, dtype=torch.bfloat16)
            self.lora_B[adapter_index] = fused_b.to(device=self.lora_B.device, dtype=torch.bfloat16)

    @staticmethod
    def fuse(*arrays: torch.Tensor, group_sizes: tuple[int, ...]) -> torch.Tensor:
        """Interleave per-component arrays group by group (inverse of ``split``)."""
        if len(arrays) != len(group_sizes):
            raise ValueError(f"got {len(arrays)} arrays but {len(group_sizes)} group_sizes")
        batch = arrays[0].shape[:-1]
        num_groups = arrays[0].shape[-1] // group_sizes[0]
        for arr, g in zip(arrays, group_sizes):
            if arr.shape[-1] != num_groups * g:
                raise ValueError(f"array last dim {arr.shape[-1]} != num_groups({num_groups}) * group_size({g})")
        parts = [arr.reshape(*batch, num_groups, g) for arr, g in zip(arrays, group_sizes)]
        return torch.cat(parts, dim=-1).reshape(*batch, -1)

    @staticmethod
    def split(fused: torch.Tensor, group_sizes: tuple[int, ...]) -> tuple[torch.Tensor, ...]:
        """Undo the group interleaving: one tensor per component."""
        batch, total = fused.shape[:-1], fused.shape[-1]
        gs = sum(group_sizes)
        if total % gs:
            raise ValueError(f"last dim {total} not divisible by sum(group_sizes)={gs}")
        num_groups = total // gs
        view = fused.reshape(*batch, num_groups, gs)
        out, offset = [], 0
        for g in group_sizes:
            out.append(view[..., offset:offset + g].reshape(*batch, num_groups * g))
            offset += g
        return tuple(out)


class LoRAExpert(LoRAMixin):
    """Expert layer (ragged per-expert linear) with multi-adapter LoRA (lora.py:354-444).

    Rows of ``x`` arrive sorted by expert; ``group_sizes[e]`` rows belong to expert ``e``.  LoRA
    pairs are indexed ``expert * max_lora_adapters + adapter`` (lora.py:414-431): rows are
    stably re-sorted by that combined index, run through the grouped kernel with
    ``max_lora_adapters`` LoRA groups per expert weight, and put back.  Differentiable: the backward
    is one native grouped call for all experts and adapters.
    """

    def __init__(self, num_experts: int, in_features: int, out_features: int, *,
                 weight: w8.PackedGroupedW8Weight | None = None, max_lora_adapters: int = 0,
                 max_lora_rank: int = 8, device="cuda:0", **_unused_reference_keywords):
        self.num_experts, self.in_features, self.out_features = int(num_experts), int(in_features), int(out_features)
        self.device = torch.device(device)
        self.weight = weight
        self.init_lora(max_lora_adapters=max_lora_adapters, max_lora_rank=max_lora_rank,
                       shape_A=(max_lora_adapters, num_experts, in_features, max_lora_rank),
                       shape_B=(max_lora_adapters, num_experts, max_lora_rank, out_features), device=self.device)

    def load_quantized(self, codes: torch.Tensor, scales: torch.Tensor) -> None:
        """int8 codes [E, in, out] and float32 scales [E, out]."""
        if tuple(codes.shape) != (self.num_experts, self.in_features, self.out_features):
            raise ValueError(f"codes must be {(self.num_experts, self.in_features, self.out_features)}")
        self.weight = w8.prepare_grouped_weight(codes.to(self.device), scales.to(self.device))

    def __call__(self, x: torch.Tensor, group_sizes: torch.Tensor, adapter_indices_sorted: torch.Tensor | None = None,
                 *, group_offset: torch.Tensor | None = None) -> torch.Tensor:
        if self.weight is None:
            raise RuntimeError("the expert kernels are not loaded: call load_quantized()")
        if group_offset is not None and int(torch.as_tensor(group_offset).reshape(-1)[0]) != 0:
            raise NotImplementedError("expert shards (group_offset != 0) belong to the multi-GPU dispatch, "
                                      "which this one-GPU build leaves out")
        if not self._lora_active(adapter_indices_sorted):
            return w8.grouped_lora_linear(x, group_sizes, self.weight)
        n_ad, n_exp = self.max_lora_adapters, self.num_experts
        gs = group_sizes.to(device=x.device, dtype=torch.int64)
        rows = torch.arange(x.shape[0], device=x.device)
        ends = torch.cumsum(gs, 0)
        # Expert of every row.  Rows beyond sum(group_sizes) belong to no expert: they sort behind every
        # group and come out as zeros, as in the plain path.  (The reference's jnp.repeat with
        # total_repeat_length, layers/lora.py:411, hands such padding rows to the last expert's adapter
        # on top of a zero base; callers drop those rows either way.)
        expert = torch.searchsorted(ends, rows, right=True)
        spare = expert >= n_exp
        adapter = adapter_indices_sorted.to(device=x.device, dtype=torch.int64).clamp(0, n_ad - 1)
        combined = torch.where(spare, n_exp * n_ad, expert * n_ad + adapter)
        order = torch.sort(combined, stable=True).indices
        sizes = torch.bincount(combined, minlength=n_exp * n_ad + 1)[: n_exp * n_ad].to(torch.int32)
        # expert-first flattening of the LoRA pairs (lora.py:418-431)
        a = self.lora_A.transpose(0, 1).reshape(n_exp * n_ad, self.in_features, self.max_lora_rank)
        b = self.lora_B.transpose(0, 1).reshape(n_exp * n_ad, self.max_lora_rank, self.out_features)
        scaling = self.lora_scaling.repeat(n_exp)
        out_sorted = w8.grouped_lora_linear(x[order], sizes, self.weight, a.contiguous(), b.contiguous(), scaling,
                                            groups_per_weight=n_ad)
        return torch.zeros_like(out_sorted).index_copy(0, order, out_sorted)


def init_lora_adapter(layer: LoRAMixin, adapter_index: int, *, rank: int, alpha: float, seed: int = 0) -> None:
    """Initialise one adapter for training (skyrl/tx/layers/lora.py:447-501): scaling = alpha /
    rank, A he-uniform with the columns at and beyond ``rank`` zeroed, B zeros.  For expert layers
    the effective rank is ``max(1, rank // num_experts)`` (lora.py:471-475)."""
    if layer.max_lora_adapters == 0:
        raise RuntimeError("the layer was built without LoRA adapters")
    if not 0 <= adapter_index < layer.max_lora_adapters:
        raise ValueError(f"adapter_index {adapter_index} outside [0, {layer.max_lora_adapters})")
    effective = max(1, rank // layer.num_experts) if isinstance(layer, LoRAExpert) else rank
    if effective > layer.max_lora_rank:
        raise ValueError(f"rank {effective} exceeds max_lora_rank {layer.max_lora_rank}")
    layer.lora_scaling[adapter_index] = alpha / effective
    layer.lora_ranks[adapter_index] = effective
    shape = layer.lora_A[adapter_index].shape
    # he_uniform as jax.nn.initializers computes it (in_axis = -2, out_axis = -1): leading axes count
    # as receptive field, so an expert layer's [E, in, r] slice has fan_in = E * in
    fan_in = math.prod(shape) // shape[-1]
    bound = math.sqrt(6.0 / fan_in)
    gen = torch.Generator(device="cpu").manual_seed(seed)
    a = (torch.rand(shape, generator=gen, dtype=torch.float32) * 2.0 - 1.0) * bound
    a[..., effective:] = 0.0
    layer.lora_A[adapter_index] = a.to(device=layer.lora_A.device, dtype=torch.bfloat16)
    layer.lora_B[adapter_index] = 0
