"""W8A8 + LoRA forward entry points on the gfx950 HIP kernels.

Keeps the call surface of the reference's ``skyrl/tx/kernels/rocm/w8a8_lora.py``
(``w8a8_frozen_linear`` :827-867, ``w8a8_lora_linear`` :870-920): explicit opt-in
with an exact ``bool``, ``TypeError`` for dtype problems, ``ValueError`` for
geometry problems, tile keywords accepted (tuning is internal, they are validated
and otherwise ignored).  Differences, all widenings: per-token / per-channel scales
(``group_size == K``) instead of group 64, any rank up to 64, float32 or bf16
scales, and an optional per-row ``adapter_indices`` with stacked adapters
(``skyrl/tx/layers/lora.py:118-157``).  ``w8a8_rms_gate_up_lora_swiglu`` and
``w8a8_lora_residual`` are the W8A8 forms of
``bf16_rms_gate_up_lora_swiglu_contiguous`` (…_contiguous.py:698-712) and
``bf16_lora_residual`` (bf16_lora_residual.py:507-522).

Tensors are torch CUDA (ROCm) tensors; kernels are enqueued on torch's current
stream.  There is no CPU or eager fallback.
"""

from __future__ import annotations

import ctypes
import functools
import math
import threading
import weakref
from dataclasses import dataclass

import torch

from .. import quantized_lora as ql
from ... import _native

DEFAULT_BLOCK_M = 32
DEFAULT_BLOCK_N = 64
DEFAULT_ROW_SUPERBLOCK = 512
MAX_BLOCK_M = 64
MAX_BLOCK_N = 128
MAX_ROW_SUPERBLOCK = 2048
MAX_IN_FEATURES = 16384
MAX_OUT_FEATURES = 1 << 20
MAX_LORA_RANK = 64
MAX_ADAPTERS = 64
_SUPPORTED_BLOCK_SIZES = frozenset((16, 32, 64, 128))


@dataclass(frozen=True)
class PackedW8Weight:
    """A [K, N] int8 weight in MFMA fragment order plus float32 per-channel scales."""

    packed: torch.Tensor   # uint8, mi355_w8a8_packed_weight_bytes(K, N)
    scales: torch.Tensor   # float32 [N]
    in_features: int
    out_features: int


def _validate_exact_bool(name: str, value) -> None:
    if type(value) is not bool:
        raise TypeError(f"{name} must be an exact bool")


def _validate_block_size(name: str, value, maximum: int) -> None:
    if isinstance(value, bool) or not isinstance(value, int):
        raise TypeError(f"{name} must be an integer")
    if value not in _SUPPORTED_BLOCK_SIZES or value > maximum:
        allowed = sorted(s for s in _SUPPORTED_BLOCK_SIZES if s <= maximum)
        raise ValueError(f"{name} must be one of {allowed}, got {value}")


def _validate_row_superblock(value, block_m: int) -> None:
    if isinstance(value, bool) or not isinstance(value, int):
        raise TypeError("row_superblock must be an integer")
    if not block_m <= value <= MAX_ROW_SUPERBLOCK:
        raise ValueError(f"row_superblock must be in [{block_m}, {MAX_ROW_SUPERBLOCK}], got {value}")
    if value % block_m:
        raise ValueError("row_superblock must be divisible by block_m")


def _stream_ptr(device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


def _version_of(t: torch.Tensor):
    """The tensor's version counter, or None where torch keeps none (tensors made under
    ``torch.inference_mode()``): in-place writes to such a tensor cannot be seen."""
    try:
        return t._version
    except RuntimeError:
        return None


def _require_cuda(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must live on the GPU (there is no CPU path); got device {t.device}")


# ---------------------------------------------------------------------------------------
# weight preparation (one time per weight)
# ---------------------------------------------------------------------------------------
_pack_cache: dict = {}
_pack_lock = threading.Lock()


def prepare_weight(weight) -> PackedW8Weight:
    """Re-layout a per-channel W8 ``GroupQuantizedWeight`` for the kernels (cached).

    This is the load-time permutation; it must not run per forward, so the result
    is cached on the identity of the codes tensor.
    """
    if isinstance(weight, PackedW8Weight):
        return weight
    ql.validate_quantized_weight(weight)
    if weight.bits != 8:
        raise ValueError(f"the native path requires W8 codes, got W{weight.bits}")
    if weight.original_in_features != weight.padded_in_features:
        raise ValueError("the native path does not accept padded K dimensions")
    if weight.group_size != weight.original_in_features:
        raise ValueError(
            f"the native path requires per-channel scales (group size {weight.original_in_features}), "
            f"got {weight.group_size}")
    k, n = weight.codes.shape
    if k % 8:
        raise ValueError("K must be a positive multiple of 8")
    if k > MAX_IN_FEATURES:
        raise ValueError(f"K must not exceed {MAX_IN_FEATURES}")
    if n > MAX_OUT_FEATURES:
        raise ValueError(f"N must not exceed {MAX_OUT_FEATURES}")
    _require_cuda(weight.codes, "weight codes")
    # (inference tensors have no version counter: they are keyed by identity and storage alone)
    key = (weight.codes.data_ptr(), weight.scales.data_ptr(), k, n, _version_of(weight.codes), _version_of(weight.scales))
    with _pack_lock:
        hit = _pack_cache.get(key)
        if hit is not None and hit[0]() is weight.codes:
            return hit[1]
    lib = _native.load()
    codes = weight.codes.contiguous()
    nbytes = int(lib.mi355_w8a8_packed_weight_bytes(k, n))
    packed = torch.empty(nbytes, dtype=torch.uint8, device=codes.device)
    with torch.cuda.device(codes.device):
        _native.check("mi355_w8a8_pack_weight_v1",
                      lib.mi355_w8a8_pack_weight_v1(codes.data_ptr(), packed.data_ptr(), k, n,
                                                    _stream_ptr(codes.device)))
    scales = weight.scales.to(torch.float32).reshape(n).contiguous()
    out = PackedW8Weight(packed=packed, scales=scales, in_features=k, out_features=n)
    with _pack_lock:
        if len(_pack_cache) > 4096:
            _pack_cache.clear()
        _pack_cache[key] = (weakref.ref(weight.codes), out)
    return out


def unpack_weight(packed: PackedW8Weight) -> torch.Tensor:
    """Inverse of the fragment-order packing: int8 [K, N] row-major."""
    lib = _native.load()
    out = torch.empty((packed.in_features, packed.out_features), dtype=torch.int8, device=packed.packed.device)
    with torch.cuda.device(out.device):
        _native.check("mi355_w8a8_unpack_weight_v1",
                      lib.mi355_w8a8_unpack_weight_v1(packed.packed.data_ptr(), out.data_ptr(),
                                                      packed.in_features, packed.out_features,
                                                      _stream_ptr(out.device)))
    return out


def dynamic_quantize_rows(x: torch.Tensor):
    """Per-token symmetric int8 quantization: (codes int8 [..., K], scales float32 [...])."""
    if x.dtype != torch.bfloat16:
        raise TypeError(f"x must be BF16, got {x.dtype}")
    if x.ndim < 2 or math.prod(x.shape[:-1]) <= 0:
        raise ValueError(f"x must have a nonempty row domain and final K axis, got {tuple(x.shape)}")
    _require_cuda(x, "x")
    lib = _native.load()
    flat = x.reshape(-1, x.shape[-1]).contiguous()
    m, k = flat.shape
    if k % 8 or k > MAX_IN_FEATURES:
        raise ValueError(f"K must be a multiple of 8 not exceeding {MAX_IN_FEATURES}, got {k}")
    codes = torch.empty((m, k), dtype=torch.int8, device=x.device)
    scales = torch.empty((m,), dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        _native.check("mi355_w8a8_quantize_rows_v1",
                      lib.mi355_w8a8_quantize_rows_v1(flat.data_ptr(), codes.data_ptr(), scales.data_ptr(),
                                                      m, k, _stream_ptr(x.device)))
    return codes.reshape(x.shape), scales.reshape(x.shape[:-1])


# ---------------------------------------------------------------------------------------
# the forward call
# ---------------------------------------------------------------------------------------

def _new_constant(value: float, count: int, device: str) -> torch.Tensor:
    # An ordinary tensor whatever mode the caller is in: a tensor created under inference_mode could
    # never be saved for a later backward.
    with torch.inference_mode(False), torch.no_grad():
        return torch.full((count,), value, dtype=torch.float32, device=torch.device(device))


_cached_constant = functools.lru_cache(maxsize=256)(_new_constant)


def _constant_scaling(value: float, count: int, device: str) -> torch.Tensor:
    """One constant vector per (value, count, device).  During a stream capture the cache is bypassed:
    a tensor created there lives in the graph's private pool, is only filled at replay and dangles once
    the graph is gone."""
    if torch.cuda.is_available() and torch.cuda.is_current_stream_capturing():
        return _new_constant(value, count, device)
    return _cached_constant(value, count, device)


def _scaling_vector(lora_scaling, count: int, device) -> torch.Tensor:
    """FP32 [count] on ``device``.  A Python number becomes one cached constant vector per (value, count,
    device): converting it at every call would be a host-to-device copy the host has to wait for, in
    front of every native call.  The cached vectors are inputs only; nothing writes them."""
    if isinstance(lora_scaling, (int, float)) and not isinstance(lora_scaling, bool):
        return _constant_scaling(float(lora_scaling), count, str(device))
    s = torch.as_tensor(lora_scaling, dtype=torch.float32, device=device)
    if s.ndim == 0:
        s = s.reshape(1).expand(count)
    return s.contiguous()


def _scaling_scalar(lora_scaling, device) -> torch.Tensor:
    """FP32 tensor on ``device`` for the autograd functions; a Python number comes from the constant cache."""
    if isinstance(lora_scaling, (int, float)) and not isinstance(lora_scaling, bool):
        return _constant_scaling(float(lora_scaling), 1, str(device)).reshape(())
    return torch.as_tensor(lora_scaling, dtype=torch.float32, device=device)


def _normalize_lora(lora_a, lora_b, lora_scaling, k: int, n: int, device):
    """Return stacked (A [n_ad,K,r], B [n_ad,r,N], s [n_ad]) bf16/bf16/f32 tensors."""
    if lora_a is None and lora_b is None:
        return None, None, None, 0, 0
    if lora_a is None or lora_b is None:
        raise ValueError("lora_a and lora_b must be given together")
    if lora_a.dtype != torch.bfloat16 or lora_b.dtype != torch.bfloat16:
        raise TypeError("LoRA A and B must both be BF16")
    if lora_a.ndim != lora_b.ndim or lora_a.ndim not in (2, 3):
        raise ValueError("lora_a and lora_b must both be rank-two, or both rank-three (stacked adapters)")
    a3 = lora_a if lora_a.ndim == 3 else lora_a[None]
    b3 = lora_b if lora_b.ndim == 3 else lora_b[None]
    n_ad, ka, r = a3.shape
    if ka != k or tuple(b3.shape) != (n_ad, r, n):
        raise ValueError(
            f"incompatible LoRA shapes: A={tuple(lora_a.shape)}, B={tuple(lora_b.shape)}, weight [K={k}, N={n}]")
    if r < 1 or r > MAX_LORA_RANK:
        raise ValueError(f"LoRA rank must be in [1, {MAX_LORA_RANK}], got {r}")
    if n_ad > MAX_ADAPTERS:
        raise ValueError(f"at most {MAX_ADAPTERS} adapters are supported, got {n_ad}")
    s = _scaling_vector(lora_scaling, n_ad, device)
    if tuple(s.shape) != (n_ad,):
        raise ValueError(f"lora_scaling must be a scalar or have shape ({n_ad},), got {tuple(s.shape)}")
    return a3.contiguous(), b3.contiguous(), s, n_ad, r


class ForwardPlan:
    """Validated arguments, output, workspace and the C struct of one forward call.

    Building the plan does all host-side checks and allocations once; ``run()`` is a
    single C call that enqueues the kernels on torch's current stream, so a caller
    that repeats the same call (a decode loop, a benchmark) pays no per-call Python
    or allocator work.  The plan keeps every tensor it points at alive.
    """

    def __init__(self, x: torch.Tensor, weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                 adapter_indices: torch.Tensor | None = None, rms_gamma: torch.Tensor | None = None,
                 eps: float = 1e-6, residual: torch.Tensor | None = None, swiglu: bool = False,
                 flags: int = 0, return_aux: bool = False, entry: str = "forward",
                 want_normalized: bool = False):
        if x.dtype != torch.bfloat16:
            raise TypeError(f"x must be BF16, got {x.dtype}")
        if x.ndim < 2 or math.prod(x.shape[:-1]) <= 0:
            raise ValueError(f"x must have a nonempty row domain and final K axis, got {tuple(x.shape)}")
        _require_cuda(x, "x")
        pw = prepare_weight(weight)
        k, n = pw.in_features, pw.out_features
        if x.shape[-1] != k:
            raise ValueError(f"x K={x.shape[-1]} does not match W8 K={k}")
        dev = x.device
        flat = x.reshape(-1, k).contiguous()
        m = flat.shape[0]
        a3, b3, s1, n_ad, r = _normalize_lora(lora_a, lora_b, lora_scaling, k, n, dev)
        idx = None
        if adapter_indices is not None:
            if n_ad == 0:
                raise ValueError("adapter_indices given without LoRA parameters")
            idx = adapter_indices.reshape(-1)
            if idx.shape[0] != m:
                if idx.shape[0] == 0 or m % idx.shape[0]:
                    raise ValueError(f"adapter_indices of length {idx.shape[0]} do not divide {m} rows")
                idx = idx.repeat_interleave(m // idx.shape[0])  # one entry per example (lora.py:142)
            idx = idx.to(device=dev, dtype=torch.int32).contiguous()
        gamma = None
        if rms_gamma is not None:
            if tuple(rms_gamma.shape) != (k,):
                raise ValueError(f"rms weight must have shape ({k},), got {tuple(rms_gamma.shape)}")
            gamma = rms_gamma.to(device=dev, dtype=torch.float32).contiguous()
        if swiglu and n % 2:
            raise ValueError("SwiGLU needs an even number of fused gate/up columns")
        n_out = n // 2 if swiglu else n
        res = None
        if residual is not None:
            if residual.dtype != torch.bfloat16:
                raise TypeError("residual must be BF16")
            if tuple(residual.shape) != (*x.shape[:-1], n_out):
                raise ValueError(
                    f"residual must have shape {(*x.shape[:-1], n_out)}, got {tuple(residual.shape)}")
            res = residual.reshape(m, n_out).contiguous()

        lib = _native.load()
        if swiglu:
            flags |= _native.FLAG_SWIGLU
        out = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
        ws_bytes = int(lib.mi355_w8a8_workspace_bytes(m, k, n, n_ad, r, flags))
        if ws_bytes == 0:
            raise ValueError(
                f"geometry M={m}, K={k}, N={n}, rank={r}, adapters={n_ad} is outside the native path")
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        aux = {}
        if return_aux:
            aux["x_codes"] = torch.empty((m, k), dtype=torch.int8, device=dev)
            aux["x_scales"] = torch.empty((m,), dtype=torch.float32, device=dev)
            aux["acc"] = torch.empty((m, n), dtype=torch.int32, device=dev)
        if (return_aux or want_normalized) and gamma is not None:
            aux["normalized"] = torch.empty((m, k), dtype=torch.bfloat16, device=dev)

        p = _native.Problem()
        p.struct_size = ctypes.sizeof(_native.Problem)
        p.flags = flags
        p.m, p.k, p.n, p.n_adapters, p.rank = m, k, n, n_ad, r
        p.rms_eps = float(eps)
        p.x = flat.data_ptr()
        p.w_packed = pw.packed.data_ptr()
        p.w_scales = pw.scales.data_ptr()
        p.lora_a = a3.data_ptr() if n_ad else None
        p.lora_b = b3.data_ptr() if n_ad else None
        p.lora_scaling = s1.data_ptr() if n_ad else None
        p.adapter_indices = idx.data_ptr() if idx is not None else None
        p.rms_gamma = gamma.data_ptr() if gamma is not None else None
        p.residual = res.data_ptr() if res is not None else None
        p.out = out.data_ptr()
        p.workspace = ws.data_ptr()
        p.workspace_bytes = ws_bytes
        p.aux_x_codes = aux["x_codes"].data_ptr() if return_aux else None
        p.aux_x_scales = aux["x_scales"].data_ptr() if return_aux else None
        p.aux_acc = aux["acc"].data_ptr() if return_aux else None
        p.aux_normalized = aux["normalized"].data_ptr() if "normalized" in aux else None
        self.problem = p
        self.device = dev
        self.entry = entry
        self.flags = flags
        self.aux = aux
        self.out = out
        self.out_shape = (*x.shape[:-1], n_out)
        self.dims = {"m": m, "k": k, "n": n, "n_out": n_out, "n_adapters": n_ad, "rank": r}
        self._fn = {"forward": lib.mi355_w8a8_forward_v1, "linear": lib.mi355_w8a8_lora_linear_v1,
                    "gateup": lib.mi355_w8a8_rms_gateup_swiglu_v1,
                    "residual": lib.mi355_w8a8_lora_residual_v1}[entry]
        self.x_flat, self.gamma, self.adapter_indices = flat, gamma, idx
        self._keep = (flat, pw, a3, b3, s1, idx, gamma, res, ws)
        self._lora = (a3, b3) if n_ad else None
        self._packed_lora_key = None  # versions of A / B whose transposed / packed copies sit in the workspace
        self.keep_lora_pack = True    # False: pack on every run (what a caller that rewrites A / B behind torch's back needs)

    def run(self, extra_flags: int = 0) -> torch.Tensor:
        """Enqueue the call on torch's current stream; returns the (reused) output tensor.

        The transposed LoRA A and packed LoRA B (for a decode-sized call: B regrouped per row by its adapter)
        live in the plan's workspace: while neither tensor nor the adapter indices have been
        written since the last full run (``Tensor._version``), the call is told to keep them
        (``FLAG_LORA_PACK_VALID``) instead of packing 2 * n * r * (K + N) bytes again.  A training step
        updates the adapters, so its forward packs once per step as before."""
        flags = self.flags | extra_flags
        key = None
        # (a captured call is replayed later, when the adapters may have changed: it always packs)
        capturing = torch.cuda.is_current_stream_capturing()
        if self._lora is not None and not capturing and self.keep_lora_pack:
            # (what the workspace holds also depends on the path the flags choose: decode kernels keep B
            # regrouped per row, the tiled kernels A and B in operand order)
            versions = (_version_of(self._lora[0]), _version_of(self._lora[1]),
                        0 if self.adapter_indices is None else _version_of(self.adapter_indices))
            if None not in versions:  # (a tensor torch keeps no version of may have been written: pack)
                key = versions + (flags & ~(_native.FLAG_SKIP_PROLOGUE | _native.FLAG_SKIP_GEMM |
                                            _native.FLAG_LORA_PACK_VALID),)
            if key is not None and key == self._packed_lora_key:
                flags |= _native.FLAG_LORA_PACK_VALID
        self.problem.flags = flags
        with torch.cuda.device(self.device):
            status = self._fn(ctypes.byref(self.problem), _stream_ptr(self.device))
        self.problem.flags = self.flags
        _native.check(f"mi355_w8a8_{self.entry}", status)
        if not extra_flags & _native.FLAG_SKIP_PROLOGUE and not capturing:
            self._packed_lora_key = key
        return self.out.reshape(self.out_shape)


def forward(x: torch.Tensor, weight, lora_a=None, lora_b=None, lora_scaling=None, *,
            adapter_indices: torch.Tensor | None = None, rms_gamma: torch.Tensor | None = None,
            eps: float = 1e-6, residual: torch.Tensor | None = None, swiglu: bool = False,
            flags: int = 0, return_aux: bool = False, entry: str = "forward"):
    """One W8A8 forward through the C ABI.  Returns bf16 [..., n_out] (and aux tensors)."""
    plan = ForwardPlan(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                       rms_gamma=rms_gamma, eps=eps, residual=residual, swiglu=swiglu, flags=flags,
                       return_aux=return_aux, entry=entry)
    result = plan.run()
    # Everything the kernels touch was allocated for torch's current stream, the one they were
    # enqueued on, so the caching allocator orders any reuse after them.
    return (result, plan.aux) if return_aux else result


# ---------------------------------------------------------------------------------------
# backward of the plain linear (skyrl/tx/kernels/quantized_lora.py:337-394)
# ---------------------------------------------------------------------------------------

class BackwardPlan:
    """Validated arguments, outputs, workspace and the C struct of one backward call; ``run()`` is
    a single C call on torch's current stream (see ``ForwardPlan``)."""

    def __init__(self, x: torch.Tensor | None, dy: torch.Tensor, weight, lora_a=None, lora_b=None,
                 lora_scaling=None, *, adapter_indices: torch.Tensor | None = None, need_lora_grads: bool = True):
        if dy.dtype != torch.bfloat16:
            raise TypeError(f"dy must be BF16, got {dy.dtype}")
        if dy.ndim < 2 or math.prod(dy.shape[:-1]) <= 0:
            raise ValueError(f"dy must have a nonempty row domain and final N axis, got {tuple(dy.shape)}")
        _require_cuda(dy, "dy")
        pw = prepare_weight(weight)
        k, n = pw.in_features, pw.out_features
        if dy.shape[-1] != n:
            raise ValueError(f"dy N={dy.shape[-1]} does not match W8 N={n}")
        dev = dy.device
        dyf = dy.reshape(-1, n).contiguous()
        m = dyf.shape[0]
        a3, b3, s1, n_ad, r = _normalize_lora(lora_a, lora_b, lora_scaling, k, n, dev)
        want = bool(n_ad) and need_lora_grads
        xf = None
        if want:
            if x is None:
                raise ValueError("x is needed for the LoRA cotangents")
            if x.dtype != torch.bfloat16:
                raise TypeError(f"x must be BF16, got {x.dtype}")
            _require_cuda(x, "x")
            if tuple(x.shape) != (*dy.shape[:-1], k):
                raise ValueError(f"x must have shape {(*dy.shape[:-1], k)}, got {tuple(x.shape)}")
            xf = x.reshape(m, k).contiguous()
        idx = None
        if adapter_indices is not None:
            if n_ad == 0:
                raise ValueError("adapter_indices given without LoRA parameters")
            idx = adapter_indices.reshape(-1)
            if idx.shape[0] != m:
                if idx.shape[0] == 0 or m % idx.shape[0]:
                    raise ValueError(f"adapter_indices of length {idx.shape[0]} do not divide {m} rows")
                idx = idx.repeat_interleave(m // idx.shape[0])
            idx = idx.to(device=dev, dtype=torch.int32).contiguous()
        lib = _native.load()
        ws_bytes = int(lib.mi355_w8a8_bwd_workspace_bytes(m, k, n, n_ad, r, 0))
        if ws_bytes == 0:
            raise ValueError(
                f"geometry M={m}, K={k}, N={n}, rank={r}, adapters={n_ad} is outside the native backward")
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        self.dx = torch.empty((m, k), dtype=torch.bfloat16, device=dev)
        self.d_lora_a = torch.empty((n_ad, k, r), dtype=torch.bfloat16, device=dev) if want else None
        self.d_lora_b = torch.empty((n_ad, r, n), dtype=torch.bfloat16, device=dev) if want else None
        self.d_lora_scaling = torch.empty((n_ad,), dtype=torch.float32, device=dev) if want else None
        p = _native.BwdProblem()
        p.struct_size = ctypes.sizeof(_native.BwdProblem)
        p.m, p.k, p.n, p.n_adapters, p.rank = m, k, n, n_ad, r
        p.x = xf.data_ptr() if xf is not None else None
        p.dy = dyf.data_ptr()
        p.w_packed = pw.packed.data_ptr()
        p.w_scales = pw.scales.data_ptr()
        p.lora_a = a3.data_ptr() if n_ad else None
        p.lora_b = b3.data_ptr() if n_ad else None
        p.lora_scaling = s1.data_ptr() if n_ad else None
        p.adapter_indices = idx.data_ptr() if idx is not None else None
        p.dx = self.dx.data_ptr()
        p.d_lora_a = self.d_lora_a.data_ptr() if want else None
        p.d_lora_b = self.d_lora_b.data_ptr() if want else None
        p.d_lora_scaling = self.d_lora_scaling.data_ptr() if want else None
        p.workspace = ws.data_ptr()
        p.workspace_bytes = ws_bytes
        self.problem = p
        self.device = dev
        self.dx_shape = (*dy.shape[:-1], k)
        self.dims = {"m": m, "k": k, "n": n, "n_adapters": n_ad, "rank": r}
        self._fn = lib.mi355_w8a8_lora_linear_bwd_v1
        self._keep = (xf, dyf, pw, a3, b3, s1, idx, ws)

    def run(self, flags: int = 0):
        """Enqueue the call; returns ``(dx, d_lora_a, d_lora_b, d_lora_scaling)`` (reused tensors)."""
        self.problem.flags = flags
        with torch.cuda.device(self.device):
            status = self._fn(ctypes.byref(self.problem), _stream_ptr(self.device))
        self.problem.flags = 0
        _native.check("mi355_w8a8_lora_linear_bwd_v1", status)
        return self.dx.reshape(self.dx_shape), self.d_lora_a, self.d_lora_b, self.d_lora_scaling


def backward(x: torch.Tensor | None, dy: torch.Tensor, weight, lora_a=None, lora_b=None, lora_scaling=None, *,
             adapter_indices: torch.Tensor | None = None, need_lora_grads: bool = True):
    """Cotangents of ``forward(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=...)``.

    Returns ``(dx, d_lora_a, d_lora_b, d_lora_scaling)``; the LoRA entries are ``None`` without
    LoRA or with ``need_lora_grads=False``.  The activation quantizer is straight-through; the
    frozen weight enters as ``bf16(codes * scales)`` (skyrl/tx/kernels/rocm/w8a8_lora.py:298-339).
    """
    return BackwardPlan(x, dy, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                        need_lora_grads=need_lora_grads).run()


class _LoraLinearFunction(torch.autograd.Function):
    """``forward`` with the custom derivative of the reference (``_quantized_lora_linear.defvjp``,
    skyrl/tx/kernels/quantized_lora.py:397): cotangents for x, A, B and the scaling; the frozen
    codes and scales get none.  With a residual (added in the float32 epilogue) its cotangent is the
    output cotangent, as in ``_bf16_lora_residual_bwd``."""

    @staticmethod
    def forward(ctx, x, lora_a, lora_b, lora_scaling, weight, adapter_indices, residual):
        out = forward(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                      residual=residual, entry="linear" if residual is None else "residual")
        ctx.save_for_backward(x, lora_a, lora_b, lora_scaling)
        ctx.weight = weight
        ctx.adapter_indices = adapter_indices
        ctx.has_residual = residual is not None
        return out

    @staticmethod
    def backward(ctx, dy):
        x, lora_a, lora_b, lora_scaling = ctx.saved_tensors
        need = lora_a is not None and any(ctx.needs_input_grad[1:4])
        dx, da, db, ds = backward(x, dy.contiguous(), ctx.weight, lora_a, lora_b, lora_scaling,
                                  adapter_indices=ctx.adapter_indices, need_lora_grads=need)
        if need:
            if lora_a.ndim == 2:
                da, db = da[0], db[0]
            ds = ds.reshape(lora_scaling.shape).to(lora_scaling.dtype)
        return dx, da, db, ds, None, None, (dy if ctx.has_residual else None)


def lora_linear(x: torch.Tensor, weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                adapter_indices: torch.Tensor | None = None, residual: torch.Tensor | None = None) -> torch.Tensor:
    """Plain W8A8 (+LoRA, + residual) linear that autograd can differentiate: the forward kernels,
    and the backward kernels when x, a LoRA parameter or the residual requires a gradient."""
    tensors = [t for t in (x, lora_a, lora_b, lora_scaling, residual) if isinstance(t, torch.Tensor)]
    if not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors)):
        return forward(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                       residual=residual, entry="linear" if residual is None else "residual")
    scaling = lora_scaling
    if lora_a is not None and not isinstance(scaling, torch.Tensor):
        scaling = _scaling_scalar(scaling, x.device)
    return _LoraLinearFunction.apply(x, lora_a, lora_b, scaling, weight, adapter_indices, residual)


# ---------------------------------------------------------------------------------------
# backward of the fused RMSNorm -> gate/up -> SwiGLU call
# (skyrl/tx/kernels/rocm/bf16_rms_gate_up_lora_swiglu_contiguous.py:643-689)
# ---------------------------------------------------------------------------------------
def swiglu_backward(fused: torch.Tensor, d_product: torch.Tensor, *, in_place: bool = False) -> torch.Tensor:
    """Cotangent of the interleaved projection from the cotangent of ``silu(gate) * up``
    (``_fp32_swiglu_pullback_interleaved``, :541-553).  ``fused`` bf16 [..., N], ``d_product``
    bf16 [..., N / 2]; with ``in_place`` the result overwrites ``fused``."""
    if fused.dtype != torch.bfloat16 or d_product.dtype != torch.bfloat16:
        raise TypeError("fused and d_product must be BF16")
    _require_cuda(fused, "fused")
    _require_cuda(d_product, "d_product")
    n = fused.shape[-1]
    if fused.ndim < 2 or n % 8 or tuple(d_product.shape) != (*fused.shape[:-1], n // 2):
        raise ValueError(f"need fused [..., N] with N % 8 == 0 and d_product [..., N / 2], got "
                         f"{tuple(fused.shape)} and {tuple(d_product.shape)}")
    if in_place and not fused.is_contiguous():
        raise ValueError("in_place needs a contiguous fused tensor")
    f2 = fused.reshape(-1, n).contiguous()
    d2 = d_product.reshape(-1, n // 2).contiguous()
    out = f2 if in_place else torch.empty_like(f2)
    with torch.cuda.device(fused.device):
        status = _native.load().mi355_w8a8_swiglu_bwd_v1(f2.data_ptr(), d2.data_ptr(), out.data_ptr(), f2.shape[0], n,
                                                         _stream_ptr(fused.device))
    _native.check("mi355_w8a8_swiglu_bwd_v1", status)
    return out.reshape(fused.shape)


def rms_norm_backward(x: torch.Tensor, gamma: torch.Tensor, d_normalized: torch.Tensor, *, eps: float = 1e-6,
                      in_place: bool = False) -> torch.Tensor:
    """Cotangent of x through ``bf16(x * rsqrt(mean(x^2) + eps) * gamma)`` (``_rms_norm_pullback``,
    :556-574); ``gamma`` float32 [K] is the multiplier itself.  With ``in_place`` the result
    overwrites ``d_normalized``."""
    if x.dtype != torch.bfloat16 or d_normalized.dtype != torch.bfloat16:
        raise TypeError("x and d_normalized must be BF16")
    _require_cuda(x, "x")
    _require_cuda(d_normalized, "d_normalized")
    k = x.shape[-1]
    if x.ndim < 2 or tuple(d_normalized.shape) != tuple(x.shape) or tuple(gamma.shape) != (k,):
        raise ValueError(f"need x and d_normalized [..., K] and gamma [K], got {tuple(x.shape)}, "
                         f"{tuple(d_normalized.shape)} and {tuple(gamma.shape)}")
    if not isinstance(eps, float) or not eps > 0.0:
        raise ValueError(f"eps must be a positive float, got {eps!r}")
    if in_place and not d_normalized.is_contiguous():
        raise ValueError("in_place needs a contiguous d_normalized tensor")
    x2 = x.reshape(-1, k).contiguous()
    d2 = d_normalized.reshape(-1, k).contiguous()
    g = gamma.to(device=x.device, dtype=torch.float32).contiguous()
    out = d2 if in_place else torch.empty_like(d2)
    with torch.cuda.device(x.device):
        status = _native.load().mi355_w8a8_rms_norm_bwd_v1(x2.data_ptr(), g.data_ptr(), d2.data_ptr(), out.data_ptr(),
                                                           x2.shape[0], k, eps, _stream_ptr(x.device))
    _native.check("mi355_w8a8_rms_norm_bwd_v1", status)
    return out.reshape(x.shape)


class FusedBackwardPlan:
    """Buffers and C structs of one backward of the fused RMSNorm -> gate/up -> SwiGLU call.

    The forward keeps neither the projection nor the normalized rows, so ``run()`` recomputes both
    with one forward call (no SwiGLU, normalized rows as the auxiliary output) and then runs three
    native stages: the SwiGLU pull-back in place on the projection, the linear backward on the
    normalized rows, and the RMSNorm pull-back in place on that call's dx.
    """

    def __init__(self, x: torch.Tensor, gamma: torch.Tensor, weight, lora_a, lora_b, lora_scaling,
                 d_product: torch.Tensor, *, adapter_indices: torch.Tensor | None = None, eps: float = 1e-6,
                 need_lora_grads: bool = True):
        if not isinstance(eps, float) or not eps > 0.0:
            raise ValueError(f"eps must be a positive float, got {eps!r}")
        self.fwd = ForwardPlan(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                               rms_gamma=gamma, eps=eps, want_normalized=True)
        d = self.fwd.dims
        m, k, n = d["m"], d["k"], d["n"]
        if n % 8:
            raise ValueError(f"the fused backward needs N % 8 == 0, got N={n}")
        if d_product.dtype != torch.bfloat16:
            raise TypeError(f"d_product must be BF16, got {d_product.dtype}")
        _require_cuda(d_product, "d_product")
        if tuple(d_product.shape) != (*x.shape[:-1], n // 2):
            raise ValueError(f"d_product must have shape {(*x.shape[:-1], n // 2)}, got {tuple(d_product.shape)}")
        self.d_product = d_product.reshape(m, n // 2).contiguous()
        self.x = self.fwd.x_flat
        self.gamma = self.fwd.gamma
        self.eps = eps
        idx = self.fwd.adapter_indices
        # fwd.out doubles as the projection and, after the in-place pull-back, as its cotangent
        self.bwd = BackwardPlan(self.fwd.aux["normalized"], self.fwd.out, weight, lora_a, lora_b, lora_scaling,
                                adapter_indices=idx, need_lora_grads=need_lora_grads)
        self.device = x.device
        self.dx_shape = tuple(x.shape)
        self.dims = d
        self._lib = _native.load()

    def run_swiglu_stage(self) -> None:
        d = self.dims
        with torch.cuda.device(self.device):
            status = self._lib.mi355_w8a8_swiglu_bwd_v1(self.fwd.out.data_ptr(), self.d_product.data_ptr(),
                                                        self.fwd.out.data_ptr(), d["m"], d["n"],
                                                        _stream_ptr(self.device))
        _native.check("mi355_w8a8_swiglu_bwd_v1", status)

    def run_rms_stage(self) -> None:
        d = self.dims
        with torch.cuda.device(self.device):
            status = self._lib.mi355_w8a8_rms_norm_bwd_v1(self.x.data_ptr(), self.gamma.data_ptr(),
                                                          self.bwd.dx.data_ptr(), self.bwd.dx.data_ptr(), d["m"],
                                                          d["k"], self.eps, _stream_ptr(self.device))
        _native.check("mi355_w8a8_rms_norm_bwd_v1", status)

    def run(self):
        """Enqueue the four calls; returns ``(dx, d_lora_a, d_lora_b, d_lora_scaling)`` (reused tensors)."""
        self.fwd.run()
        self.run_swiglu_stage()
        dn, da, db, ds = self.bwd.run()
        self.run_rms_stage()
        return dn.reshape(self.dx_shape), da, db, ds


def rms_gate_up_swiglu_backward(x: torch.Tensor, gamma: torch.Tensor, weight, lora_a, lora_b, lora_scaling,
                                d_product: torch.Tensor, *, adapter_indices: torch.Tensor | None = None,
                                eps: float = 1e-6, need_lora_grads: bool = True):
    """Cotangents ``(dx, d_lora_a, d_lora_b, d_lora_scaling)`` of the fused call
    (bf16_rms_gate_up_lora_swiglu_contiguous.py:643-689 around the quantized projection's own rule)."""
    return FusedBackwardPlan(x, gamma, weight, lora_a, lora_b, lora_scaling, d_product,
                             adapter_indices=adapter_indices, eps=eps, need_lora_grads=need_lora_grads).run()


def swiglu(fused: torch.Tensor) -> torch.Tensor:
    """``bf16(silu(gate) * up)`` of an interleaved bf16 projection [..., N] -> [..., N / 2], bit for bit
    what the fused forward produces (``_fp32_swiglu_from_interleaved``, :535-538)."""
    if fused.dtype != torch.bfloat16:
        raise TypeError(f"fused must be BF16, got {fused.dtype}")
    _require_cuda(fused, "fused")
    n = fused.shape[-1]
    if fused.ndim < 2 or n % 8:
        raise ValueError(f"need fused [..., N] with N % 8 == 0, got {tuple(fused.shape)}")
    f2 = fused.reshape(-1, n).contiguous()
    out = torch.empty((f2.shape[0], n // 2), dtype=torch.bfloat16, device=fused.device)
    with torch.cuda.device(fused.device):
        status = _native.load().mi355_w8a8_swiglu_v1(f2.data_ptr(), out.data_ptr(), f2.shape[0], n,
                                                     _stream_ptr(fused.device))
    _native.check("mi355_w8a8_swiglu_v1", status)
    return out.reshape(*fused.shape[:-1], n // 2)


class _RmsGateUpFunction(torch.autograd.Function):
    """The fused forward with the derivative rule of ``_bf16_rms_gate_up_lora_swiglu_contiguous``
    (bf16_rms_gate_up_lora_swiglu_contiguous.py:577-695): cotangents for x, A, B (and the scaling);
    none for the norm weight and the frozen kernel.

    With ``save_projection`` the forward keeps the bf16 projection and the normalized rows for the
    backward, as the reference's training forward does (``_forward_with_residuals``, :489-532): the
    projection runs without the SwiGLU flag and a separate kernel forms the product (bit-identical
    output).  Without it the forward keeps nothing and the backward recomputes both.
    """

    @staticmethod
    def forward(ctx, x, lora_a, lora_b, lora_scaling, gamma, weight, adapter_indices, eps, save_projection):
        ctx.weight = weight
        ctx.adapter_indices = adapter_indices
        ctx.eps = eps
        ctx.saved_projection = bool(save_projection) and prepare_weight(weight).out_features % 8 == 0
        if ctx.saved_projection:
            # the tiled kernel, as the fused call takes it (the streaming kernels for few rows have no
            # SwiGLU epilogue and add the LoRA term in another order): the product is then bit-identical
            plan = ForwardPlan(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                               rms_gamma=gamma, eps=eps, want_normalized=True, flags=_native.FLAG_FORCE_TILED)
            fused = plan.run()
            ctx.save_for_backward(x, lora_a, lora_b, lora_scaling, gamma, fused, plan.aux["normalized"])
            return swiglu(fused)
        ctx.save_for_backward(x, lora_a, lora_b, lora_scaling, gamma)
        return forward(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                       rms_gamma=gamma, eps=eps, swiglu=True, entry="gateup")

    @staticmethod
    def backward(ctx, d_product):
        x, lora_a, lora_b, lora_scaling, gamma = ctx.saved_tensors[:5]
        need = lora_a is not None and any(ctx.needs_input_grad[1:4])
        if ctx.saved_projection:
            fused, normalized = ctx.saved_tensors[5:]
            d_fused = swiglu_backward(fused, d_product.contiguous().reshape(*fused.shape[:-1], -1))
            idx = ctx.adapter_indices
            rows = normalized.shape[0]
            if idx is not None and idx.numel() != rows:
                idx = idx.reshape(-1).repeat_interleave(rows // idx.numel())
            dn, da, db, ds = backward(normalized, d_fused.reshape(rows, -1), ctx.weight, lora_a, lora_b, lora_scaling,
                                      adapter_indices=idx, need_lora_grads=need)
            dx = rms_norm_backward(x.reshape(rows, -1), gamma, dn, eps=ctx.eps, in_place=True).reshape(x.shape)
        else:
            dx, da, db, ds = rms_gate_up_swiglu_backward(x, gamma, ctx.weight, lora_a, lora_b, lora_scaling,
                                                         d_product.contiguous(),
                                                         adapter_indices=ctx.adapter_indices, eps=ctx.eps,
                                                         need_lora_grads=need)
        if need:
            if lora_a.ndim == 2:
                da, db = da[0], db[0]
            ds = ds.reshape(lora_scaling.shape).to(lora_scaling.dtype)
        return dx, da, db, ds, None, None, None, None, None


def rms_gate_up_lora_swiglu(x: torch.Tensor, gamma: torch.Tensor, weight, lora_a=None, lora_b=None,
                            lora_scaling=None, *, adapter_indices: torch.Tensor | None = None,
                            eps: float = 1e-6, save_projection: bool = True) -> torch.Tensor:
    """RMSNorm (multiplier ``gamma``, float32) -> W8A8 gate/up (+LoRA) -> SwiGLU that autograd can
    differentiate in x and the LoRA parameters.  ``save_projection`` (default, the reference's
    choice) trades 2 * M * (N + K) bytes kept until the backward for not recomputing the projection."""
    tensors = [t for t in (x, lora_a, lora_b, lora_scaling) if isinstance(t, torch.Tensor)]
    if not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors)):
        return forward(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                       rms_gamma=gamma, eps=eps, swiglu=True, entry="gateup")
    scaling = lora_scaling
    if lora_a is not None and not isinstance(scaling, torch.Tensor):
        scaling = _scaling_scalar(scaling, x.device)
    return _RmsGateUpFunction.apply(x, lora_a, lora_b, scaling, gamma, weight, adapter_indices, eps, save_projection)


# ---------------------------------------------------------------------------------------
# grouped (ragged, per-expert) variant
# ---------------------------------------------------------------------------------------
@dataclass(frozen=True, eq=False)
class PackedGroupedW8Weight:
    """E stacked [K, N] int8 weights in MFMA fragment order plus float32 scales [E, N].  Compared and hashed
    by identity (it keys the expert layer's plan cache)."""

    packed: torch.Tensor
    scales: torch.Tensor
    n_weights: int
    in_features: int
    out_features: int


def prepare_grouped_weight(codes: torch.Tensor, scales: torch.Tensor) -> PackedGroupedW8Weight:
    """Pack per-expert int8 codes [E, K, N] with per-channel scales [E, N] (or [E, 1, N]) once."""
    if codes.ndim != 3 or codes.dtype != torch.int8:
        raise TypeError("grouped W8 codes must be a rank-three INT8 array [E, K, N]")
    _require_cuda(codes, "weight codes")
    e, k, n = codes.shape
    if k % 8 or k > MAX_IN_FEATURES:
        raise ValueError(f"K must be a multiple of 8 not exceeding {MAX_IN_FEATURES}, got {k}")
    if scales.numel() != e * n or not scales.dtype.is_floating_point:
        raise ValueError(f"scales must be floating point with {e * n} elements, got {tuple(scales.shape)}")
    lib = _native.load()
    each = int(lib.mi355_w8a8_packed_weight_bytes(k, n))
    packed = torch.empty(e * each, dtype=torch.uint8, device=codes.device)
    codes = codes.contiguous()
    with torch.cuda.device(codes.device):
        for i in range(e):
            _native.check("mi355_w8a8_pack_weight_v1",
                          lib.mi355_w8a8_pack_weight_v1(codes[i].data_ptr(), packed.data_ptr() + i * each, k, n,
                                                        _stream_ptr(codes.device)))
    return PackedGroupedW8Weight(packed=packed, scales=scales.to(torch.float32).reshape(e, n).contiguous(),
                                 n_weights=e, in_features=k, out_features=n)


class GroupedForwardPlan:
    """Validated arguments, output, workspace and the C struct of one ragged W8A8 (+LoRA) call;
    ``run()`` is a single C call on torch's current stream that neither allocates nor synchronizes, so
    it can be captured in a HIP graph.  ``x``, ``group_sizes`` (``plan.group_sizes``), the LoRA tensors
    and ``row_map`` (``plan.row_map``) are read at every run: rewrite them in place between runs.

    Rows of ``x`` are sorted by group; group g owns ``group_sizes[g]`` consecutive rows and uses weight
    ``g // groups_per_weight`` and LoRA pair g.  Rows beyond ``sum(group_sizes)`` give zeros
    (``lax.ragged_dot`` semantics).

    With ``row_map`` (int32 [rows]) the call has ``row_map.numel()`` rows and row i is read from
    ``x[row_map[i] // row_repeat]``: the sorted (token, choice) pairs of an expert layer read the
    unsorted hidden states, and no sorted copy of them is ever written."""

    def __init__(self, x: torch.Tensor, group_sizes: torch.Tensor, weight: PackedGroupedW8Weight, lora_a=None,
                 lora_b=None, lora_scaling=None, *, swiglu: bool = False, groups_per_weight: int = 1,
                 flags: int = 0, return_aux: bool = False, row_map: torch.Tensor | None = None,
                 row_repeat: int = 1):
        if x.dtype != torch.bfloat16:
            raise TypeError(f"x must be BF16, got {x.dtype}")
        if x.ndim != 2 or x.shape[0] <= 0:
            raise ValueError(f"x must be [rows, K] with at least one row, got {tuple(x.shape)}")
        _require_cuda(x, "x")
        k, n = weight.in_features, weight.out_features
        if x.shape[1] != k:
            raise ValueError(f"x K={x.shape[1]} does not match W8 K={k}")
        dev = x.device
        flat = x.contiguous()
        m = flat.shape[0]
        rmap = None
        if row_map is not None:
            if isinstance(row_repeat, bool) or not isinstance(row_repeat, int) or row_repeat < 1:
                raise ValueError(f"row_repeat must be a positive integer, got {row_repeat!r}")
            rmap = row_map.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
            m = rmap.numel()
            if m <= 0 or m > flat.shape[0] * row_repeat:
                raise ValueError(f"row_map with {m} entries does not fit {flat.shape[0]} rows x {row_repeat}")
        gs = group_sizes.to(device=dev, dtype=torch.int32).contiguous()
        n_groups = gs.numel()
        if n_groups != weight.n_weights * groups_per_weight:
            raise ValueError(f"{n_groups} groups do not match {weight.n_weights} weights x {groups_per_weight}")
        a3 = b3 = s1 = None
        r = 0
        if lora_a is not None:
            if lora_a.dtype != torch.bfloat16 or lora_b.dtype != torch.bfloat16:
                raise TypeError("LoRA A and B must both be BF16")
            if lora_a.ndim != 3 or lora_b.ndim != 3 or lora_a.shape[0] != n_groups or lora_a.shape[1] != k:
                raise ValueError(f"grouped lora_a must be [{n_groups}, {k}, r], got {tuple(lora_a.shape)}")
            r = lora_a.shape[2]
            if tuple(lora_b.shape) != (n_groups, r, n):
                raise ValueError(f"grouped lora_b must be [{n_groups}, {r}, {n}], got {tuple(lora_b.shape)}")
            if r < 1 or r > MAX_LORA_RANK:
                raise ValueError(f"LoRA rank must be in [1, {MAX_LORA_RANK}], got {r}")
            a3, b3 = lora_a.contiguous(), lora_b.contiguous()
            s1 = _scaling_vector(lora_scaling, n_groups, dev)
            if tuple(s1.shape) != (n_groups,):
                raise ValueError(f"lora_scaling must be a scalar or have shape ({n_groups},)")
        if swiglu and n % 2:
            raise ValueError("SwiGLU needs an even number of fused gate/up columns")
        n_out = n // 2 if swiglu else n
        lib = _native.load()
        if swiglu:
            flags |= _native.FLAG_SWIGLU
        ws_bytes = int(lib.mi355_w8a8_grouped_workspace_bytes(m, k, n, n_groups, r, flags))
        if ws_bytes == 0:
            raise ValueError(f"geometry M={m}, K={k}, N={n}, groups={n_groups}, rank={r} is outside the native path")
        self.device = dev
        self.out = torch.empty((m, n_out), dtype=torch.bfloat16, device=dev)
        self.workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        self.aux = {}
        if return_aux:
            self.aux["x_codes"] = torch.empty((m, k), dtype=torch.int8, device=dev)
            self.aux["x_scales"] = torch.empty((m,), dtype=torch.float32, device=dev)
            self.aux["acc"] = torch.zeros((m, n), dtype=torch.int32, device=dev)
        self.x_flat, self.group_sizes, self.row_map, self.weight = flat, gs, rmap, weight
        self._keep = (a3, b3, s1)
        p = _native.GroupedProblem()
        p.struct_size = ctypes.sizeof(_native.GroupedProblem)
        p.flags = flags
        p.m, p.k, p.n, p.n_groups, p.rank, p.groups_per_weight = m, k, n, n_groups, r, groups_per_weight
        p.x = flat.data_ptr()
        p.w_packed = weight.packed.data_ptr()
        p.w_scales = weight.scales.data_ptr()
        p.lora_a = a3.data_ptr() if r else None
        p.lora_b = b3.data_ptr() if r else None
        p.lora_scaling = s1.data_ptr() if r else None
        p.group_sizes = gs.data_ptr()
        p.out = self.out.data_ptr()
        p.workspace = self.workspace.data_ptr()
        p.workspace_bytes = ws_bytes
        p.aux_x_codes = self.aux["x_codes"].data_ptr() if return_aux else None
        p.aux_x_scales = self.aux["x_scales"].data_ptr() if return_aux else None
        p.aux_acc = self.aux["acc"].data_ptr() if return_aux else None
        p.x_row_map = rmap.data_ptr() if rmap is not None else None
        p.x_row_repeat = row_repeat if rmap is not None else 0
        p.x_rows = flat.shape[0] if rmap is not None else 0
        self.problem = p
        self.flags = flags
        self._lib = lib
        self._lora = (a3, b3) if r else None
        self._packed_lora_key = None  # versions of A and B the workspace holds in operand order
        self.keep_lora_pack = True    # False: pack on every run

    def bind_x(self, x: torch.Tensor) -> None:
        """Read the rows from another tensor of the same shape from the next run on (the plan keeps it alive)."""
        if x.dtype != torch.bfloat16 or tuple(x.shape) != tuple(self.x_flat.shape) or x.device != self.device:
            raise ValueError(f"bind_x needs a BF16 tensor of shape {tuple(self.x_flat.shape)} on {self.device}")
        self.x_flat = x.contiguous()
        self.problem.x = self.x_flat.data_ptr()

    def run(self, extra_flags: int = 0) -> torch.Tensor:
        """Enqueue the call on torch's current stream; returns the (reused) output tensor.  ``extra_flags``
        adds the measurement flags ``FLAG_SKIP_PROLOGUE`` / ``FLAG_SKIP_GEMM`` for this run.

        As in ``ForwardPlan.run``: while neither adapter tensor has been written since the last full run
        (``Tensor._version``) the call keeps the operand packs in its workspace
        (``FLAG_LORA_PACK_VALID``); never under graph capture."""
        flags = self.flags | extra_flags
        key = None
        capturing = torch.cuda.is_current_stream_capturing()
        if self._lora is not None and not capturing and self.keep_lora_pack:
            versions = (_version_of(self._lora[0]), _version_of(self._lora[1]))
            if None not in versions:  # (a tensor torch keeps no version of may have been written: pack)
                key = versions + (flags & ~(_native.FLAG_SKIP_PROLOGUE | _native.FLAG_SKIP_GEMM |
                                            _native.FLAG_LORA_PACK_VALID),)
            if key is not None and key == self._packed_lora_key:
                flags |= _native.FLAG_LORA_PACK_VALID
        self.problem.flags = flags
        with torch.cuda.device(self.device):
            status = self._lib.mi355_w8a8_grouped_v1(ctypes.byref(self.problem), _stream_ptr(self.device))
        self.problem.flags = self.flags
        _native.check("mi355_w8a8_grouped_v1", status)
        if not extra_flags & _native.FLAG_SKIP_PROLOGUE and not capturing:
            self._packed_lora_key = key
        return self.out


def grouped_forward(x: torch.Tensor, group_sizes: torch.Tensor, weight: PackedGroupedW8Weight, lora_a=None,
                    lora_b=None, lora_scaling=None, *, swiglu: bool = False, groups_per_weight: int = 1,
                    flags: int = 0, return_aux: bool = False, row_map: torch.Tensor | None = None,
                    row_repeat: int = 1):
    """Ragged W8A8 (+LoRA) linear in one native call: a ``GroupedForwardPlan`` built and run once."""
    plan = GroupedForwardPlan(x, group_sizes, weight, lora_a, lora_b, lora_scaling, swiglu=swiglu,
                              groups_per_weight=groups_per_weight, flags=flags, return_aux=return_aux,
                              row_map=row_map, row_repeat=row_repeat)
    out = plan.run()
    return (out, plan.aux) if return_aux else out


class GroupedBackwardPlan:
    """Validated arguments, outputs, workspace and the C struct of one grouped backward call;
    ``run()`` is a single C call on torch's current stream.  Nothing is read back to the host."""

    def __init__(self, x: torch.Tensor | None, dy: torch.Tensor, group_sizes: torch.Tensor,
                 weight: PackedGroupedW8Weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                 groups_per_weight: int = 1, need_lora_grads: bool = True):
        if dy.ndim != 2 or dy.dtype != torch.bfloat16:
            raise TypeError("dy must be a BF16 matrix [rows, N]")
        _require_cuda(dy, "dy")
        k, n = weight.in_features, weight.out_features
        if dy.shape[1] != n or dy.shape[0] <= 0:
            raise ValueError(f"dy must be [rows, {n}] with at least one row, got {tuple(dy.shape)}")
        dev = dy.device
        dyf = dy.contiguous()
        m = dyf.shape[0]
        gpw = int(groups_per_weight)
        gs = group_sizes.to(device=dev, dtype=torch.int32).contiguous()
        n_groups = gs.numel()
        if gpw < 1 or n_groups != weight.n_weights * gpw:
            raise ValueError(f"{n_groups} groups do not match {weight.n_weights} weights x {gpw}")
        a3 = b3 = s1 = xf = None
        r = 0
        if lora_a is not None:
            if lora_a.dtype != torch.bfloat16 or lora_b.dtype != torch.bfloat16:
                raise TypeError("LoRA A and B must both be BF16")
            if lora_a.ndim != 3 or lora_a.shape[0] != n_groups or lora_a.shape[1] != k:
                raise ValueError(f"grouped lora_a must be [{n_groups}, {k}, r], got {tuple(lora_a.shape)}")
            r = lora_a.shape[2]
            if tuple(lora_b.shape) != (n_groups, r, n):
                raise ValueError(f"grouped lora_b must be [{n_groups}, {r}, {n}], got {tuple(lora_b.shape)}")
            if r < 1 or r > MAX_LORA_RANK:
                raise ValueError(f"LoRA rank must be in [1, {MAX_LORA_RANK}], got {r}")
            a3, b3 = lora_a.detach().contiguous(), lora_b.detach().contiguous()
            s1 = _scaling_vector(lora_scaling, n_groups, dev).detach()
            if tuple(s1.shape) != (n_groups,):
                raise ValueError(f"lora_scaling must be a scalar or have shape ({n_groups},)")
        want = bool(r) and need_lora_grads
        if want:
            if x is None:
                raise ValueError("x is needed for the LoRA cotangents")
            if x.dtype != torch.bfloat16 or tuple(x.shape) != (m, k):
                raise ValueError(f"x must be BF16 [{m}, {k}], got {x.dtype} {tuple(x.shape)}")
            _require_cuda(x, "x")
            xf = x.detach().contiguous()
        lib = _native.load()
        ws_bytes = int(lib.mi355_w8a8_grouped_bwd_workspace_bytes(m, k, n, n_groups, r, gpw))
        if ws_bytes == 0:
            raise ValueError(f"geometry M={m}, K={k}, N={n}, groups={n_groups}, rank={r} is outside the native backward")
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        self.dx = torch.empty((m, k), dtype=torch.bfloat16, device=dev)
        self.d_lora_a = torch.empty((n_groups, k, r), dtype=torch.bfloat16, device=dev) if want else None
        self.d_lora_b = torch.empty((n_groups, r, n), dtype=torch.bfloat16, device=dev) if want else None
        self.d_lora_scaling = torch.empty((n_groups,), dtype=torch.float32, device=dev) if want else None
        p = _native.GroupedBwdProblem()
        p.struct_size = ctypes.sizeof(_native.GroupedBwdProblem)
        p.m, p.k, p.n, p.n_groups, p.rank, p.groups_per_weight = m, k, n, n_groups, r, gpw
        p.x = xf.data_ptr() if xf is not None else None
        p.dy = dyf.data_ptr()
        p.w_packed, p.w_scales = weight.packed.data_ptr(), weight.scales.data_ptr()
        p.lora_a = a3.data_ptr() if r else None
        p.lora_b = b3.data_ptr() if r else None
        p.lora_scaling = s1.data_ptr() if r else None
        p.group_sizes = gs.data_ptr()
        p.dx = self.dx.data_ptr()
        p.d_lora_a = self.d_lora_a.data_ptr() if want else None
        p.d_lora_b = self.d_lora_b.data_ptr() if want else None
        p.d_lora_scaling = self.d_lora_scaling.data_ptr() if want else None
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws_bytes
        self.problem = p
        self.device = dev
        self.dims = {"m": m, "k": k, "n": n, "n_groups": n_groups, "rank": r}
        self.group_sizes = gs   # the int32 tensor the call reads: rewrite it in place to route the next run differently
        self._fn = lib.mi355_w8a8_grouped_bwd_v1
        self._keep = (xf, dyf, gs, weight, a3, b3, s1, ws)

    def run(self):
        """Enqueue the call; returns ``(dx, d_lora_a, d_lora_b, d_lora_scaling)`` (reused tensors)."""
        with torch.cuda.device(self.device):
            status = self._fn(ctypes.byref(self.problem), _stream_ptr(self.device))
        _native.check("mi355_w8a8_grouped_bwd_v1", status)
        return self.dx, self.d_lora_a, self.d_lora_b, self.d_lora_scaling


def grouped_backward(x: torch.Tensor | None, dy: torch.Tensor, group_sizes: torch.Tensor,
                     weight: PackedGroupedW8Weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                     groups_per_weight: int = 1, need_lora_grads: bool = True):
    """Cotangents of ``grouped_forward`` (plain epilogue): ``(dx, d_lora_a, d_lora_b, d_lora_scaling)``,
    one native call for all groups (the derivative of ``LoRAExpert.__call__``, skyrl/tx/layers/lora.py:
    394-444, under the rule of ``backward``).  Rows beyond ``sum(group_sizes)`` get a zero ``dx``;
    groups without rows get zero cotangents."""
    return GroupedBackwardPlan(x, dy, group_sizes, weight, lora_a, lora_b, lora_scaling,
                               groups_per_weight=groups_per_weight, need_lora_grads=need_lora_grads).run()


def grouped_backward_per_weight(x: torch.Tensor | None, dy: torch.Tensor, group_sizes: torch.Tensor,
                     weight: PackedGroupedW8Weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                     groups_per_weight: int = 1, need_lora_grads: bool = True):
    """The same cotangents as ``grouped_backward`` from one dense backward call per weight (expert)
    over its rows, the groups that share the weight taking the role of adapters.  The group sizes
    are read on the host to cut the rows, which waits for the stream; kept as the statement of what
    the single native call computes (the two agree bit for bit)."""
    if dy.ndim != 2 or dy.dtype != torch.bfloat16:
        raise TypeError("dy must be a BF16 matrix [rows, N]")
    _require_cuda(dy, "dy")
    k, n = weight.in_features, weight.out_features
    if dy.shape[1] != n:
        raise ValueError(f"dy N={dy.shape[1]} does not match W8 N={n}")
    gpw = int(groups_per_weight)
    sizes = [max(0, int(v)) for v in group_sizes.detach().to("cpu").reshape(-1).tolist()]
    if len(sizes) != weight.n_weights * gpw:
        raise ValueError(f"{len(sizes)} groups do not match {weight.n_weights} weights x {gpw}")
    lora = lora_a is not None
    want = lora and need_lora_grads
    dev = dy.device
    m = dy.shape[0]
    dx = torch.zeros((m, k), dtype=torch.bfloat16, device=dev)
    da = torch.zeros_like(lora_a) if want else None
    db = torch.zeros_like(lora_b) if want else None
    s_all = None
    if lora:
        s_all = torch.as_tensor(lora_scaling, dtype=torch.float32, device=dev)
        s_all = s_all.reshape(1).expand(len(sizes)).contiguous() if s_all.ndim == 0 else s_all
    ds = torch.zeros(len(sizes), dtype=torch.float32, device=dev) if want else None
    each = weight.packed.numel() // weight.n_weights
    row = 0
    for wi in range(weight.n_weights):
        g0 = wi * gpw
        counts = sizes[g0:g0 + gpw]
        rows = min(sum(counts), m - row)
        if rows <= 0:
            continue
        pw = PackedW8Weight(packed=weight.packed[wi * each:(wi + 1) * each], scales=weight.scales[wi],
                            in_features=k, out_features=n)
        sl = slice(row, row + rows)
        idx = None
        if lora and gpw > 1:
            idx = torch.repeat_interleave(torch.arange(gpw, dtype=torch.int32, device=dev),
                                          torch.tensor(counts, device=dev))[:rows]
        out = backward(x[sl] if want else None, dy[sl], pw,
                       lora_a[g0:g0 + gpw] if lora else None, lora_b[g0:g0 + gpw] if lora else None,
                       s_all[g0:g0 + gpw] if lora else None, adapter_indices=idx, need_lora_grads=want)
        dx[sl] = out[0]
        if want:
            da[g0:g0 + gpw], db[g0:g0 + gpw], ds[g0:g0 + gpw] = out[1], out[2], out[3]
        row += rows
    return dx, da, db, ds


class _GroupedLinearFunction(torch.autograd.Function):
    """``grouped_forward`` (plain epilogue) with the per-expert backward as its derivative."""

    @staticmethod
    def forward(ctx, x, lora_a, lora_b, lora_scaling, weight, group_sizes, groups_per_weight):
        out = grouped_forward(x, group_sizes, weight, lora_a, lora_b, lora_scaling,
                              groups_per_weight=groups_per_weight)
        ctx.save_for_backward(x, lora_a, lora_b, lora_scaling, group_sizes)
        ctx.weight = weight
        ctx.gpw = groups_per_weight
        return out

    @staticmethod
    def backward(ctx, dy):
        x, lora_a, lora_b, lora_scaling, group_sizes = ctx.saved_tensors
        need = lora_a is not None and any(ctx.needs_input_grad[1:4])
        dx, da, db, ds = grouped_backward(x, dy.contiguous(), group_sizes, ctx.weight, lora_a, lora_b,
                                          lora_scaling, groups_per_weight=ctx.gpw, need_lora_grads=need)
        if need:
            ds = ds.reshape(lora_scaling.shape).to(lora_scaling.dtype) if lora_scaling.ndim else ds.sum()
        return dx, da, db, ds, None, None, None


def grouped_lora_linear(x, group_sizes, weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                        groups_per_weight: int = 1):
    """Ragged W8A8 (+LoRA) linear that autograd can differentiate (plain epilogue only)."""
    tensors = [t for t in (x, lora_a, lora_b, lora_scaling) if isinstance(t, torch.Tensor)]
    if not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors)):
        return grouped_forward(x, group_sizes, weight, lora_a, lora_b, lora_scaling,
                               groups_per_weight=groups_per_weight)
    scaling = lora_scaling
    if lora_a is not None and not isinstance(scaling, torch.Tensor):
        scaling = _scaling_scalar(scaling, x.device)
    return _GroupedLinearFunction.apply(x, lora_a, lora_b, scaling, weight, group_sizes, groups_per_weight)


def w8a8_grouped_lora_linear(x, group_sizes, weight, lora_a=None, lora_b=None, lora_scaling=None, *,
                             enabled: bool = False, interpret: bool = False, swiglu: bool = False,
                             groups_per_weight: int = 1):
    """W8A8 form of ``LoRAExpert.__call__`` (skyrl/tx/layers/lora.py:394-444): per-group frozen
    weight plus per-group LoRA over rows that are already sorted by group."""
    _check_enabled(enabled, interpret, "grouped LoRA")
    return grouped_forward(x, group_sizes, weight, lora_a, lora_b, lora_scaling, swiglu=swiglu,
                           groups_per_weight=groups_per_weight)


def moe_route(router_logits: torch.Tensor, top_k: int, norm_topk_prob: bool = True):
    """softmax -> top-k -> renormalise (skyrl/tx/models/qwen3.py:175-178) in float32.  Returns
    ``(weights f32 [T, top_k], selected int32 [T, top_k])``; ties pick the lower expert."""
    _require_cuda(router_logits, "router_logits")
    if router_logits.ndim != 2 or router_logits.shape[0] <= 0:
        raise ValueError(f"router_logits must be [tokens, experts], got {tuple(router_logits.shape)}")
    if isinstance(top_k, bool) or not isinstance(top_k, int) or not 1 <= top_k <= router_logits.shape[1]:
        raise ValueError(f"top_k must be an integer in [1, {router_logits.shape[1]}], got {top_k!r}")
    _validate_exact_bool("norm_topk_prob", norm_topk_prob)
    logits = router_logits.detach().to(torch.float32).contiguous()
    t, e = logits.shape
    dev = logits.device
    weights = torch.empty((t, top_k), dtype=torch.float32, device=dev)
    selected = torch.empty((t, top_k), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        status = _native.load().mi355_w8a8_moe_route_v1(logits.data_ptr(), t, e, top_k, int(norm_topk_prob),
                                                        weights.data_ptr(), selected.data_ptr(), _stream_ptr(dev))
    _native.check("mi355_w8a8_moe_route_v1", status)
    return weights, selected


def moe_route_backward(router_logits: torch.Tensor, selected: torch.Tensor, d_weights: torch.Tensor,
                       norm_topk_prob: bool = True) -> torch.Tensor:
    """Cotangent of the router logits from the cotangent of the routing weights, the selection held
    fixed as ``lax.top_k`` does (the derivative of qwen3.py:175-178).  float32 [T, E]."""
    _require_cuda(router_logits, "router_logits")
    if router_logits.ndim != 2 or tuple(selected.shape) != tuple(d_weights.shape) or selected.ndim != 2 or \
            selected.shape[0] != router_logits.shape[0]:
        raise ValueError(f"need router_logits [T, E] and selected, d_weights [T, top_k], got "
                         f"{tuple(router_logits.shape)}, {tuple(selected.shape)}, {tuple(d_weights.shape)}")
    _validate_exact_bool("norm_topk_prob", norm_topk_prob)
    dev = router_logits.device
    logits = router_logits.detach().to(torch.float32).contiguous()
    sel = selected.to(device=dev, dtype=torch.int32).contiguous()
    dw = d_weights.detach().to(device=dev, dtype=torch.float32).contiguous()
    t, e = logits.shape
    out = torch.empty_like(logits)
    with torch.cuda.device(dev):
        status = _native.load().mi355_w8a8_moe_route_bwd_v1(logits.data_ptr(), sel.data_ptr(), dw.data_ptr(), t, e,
                                                            sel.shape[1], int(norm_topk_prob), out.data_ptr(),
                                                            _stream_ptr(dev))
    _native.check("mi355_w8a8_moe_route_bwd_v1", status)
    return out


class _MoeRouteFunction(torch.autograd.Function):
    """``moe_route`` whose weights are differentiable in the logits (the indices are not)."""

    @staticmethod
    def forward(ctx, router_logits, top_k, norm_topk_prob):
        weights, selected = moe_route(router_logits, top_k, norm_topk_prob)
        ctx.save_for_backward(router_logits, selected)
        ctx.norm = norm_topk_prob
        ctx.mark_non_differentiable(selected)
        return weights, selected

    @staticmethod
    def backward(ctx, d_weights, _d_selected):
        router_logits, selected = ctx.saved_tensors
        d_logits = moe_route_backward(router_logits, selected, d_weights.contiguous(), ctx.norm)
        return d_logits.reshape(router_logits.shape).to(router_logits.dtype), None, None


def moe_dispatch(tokens: torch.Tensor | None, indices: torch.Tensor, num_groups: int, *, repeat: int = 1,
                 adapter_indices: torch.Tensor | None = None, out=None):
    """Stable sort of rows by group with the gather of their token rows, on the device and without a
    host round trip.  Pair ``p`` reads token ``p // repeat`` (and its adapter index).  Returns
    ``(sorted_tokens, group_sizes, sort_indices, unsort_indices, sorted_adapters)``.  ``out`` names
    ``(group_sizes, sort_indices, unsort_indices, workspace)`` of an earlier call with the same sizes to write
    into instead of new tensors."""
    _require_cuda(indices, "indices")
    dev = indices.device
    idx = indices.reshape(-1).to(torch.int32).contiguous()
    n_pairs = idx.numel()
    if n_pairs <= 0:
        raise ValueError("indices must not be empty")
    if isinstance(repeat, bool) or not isinstance(repeat, int) or repeat < 1 or n_pairs % repeat:
        raise ValueError(f"repeat must be a positive integer dividing {n_pairs} rows, got {repeat!r}")
    if isinstance(num_groups, bool) or not isinstance(num_groups, int) or num_groups < 1:
        raise ValueError(f"num_groups must be a positive integer, got {num_groups!r}")
    lib = _native.load()
    ws_bytes = int(lib.mi355_w8a8_moe_dispatch_workspace_bytes(n_pairs, num_groups))
    if ws_bytes == 0:
        raise ValueError(f"{n_pairs} rows in {num_groups} groups are outside the native dispatch")
    tok = sorted_tokens = None
    width = 0
    if tokens is not None:
        if tokens.dtype != torch.bfloat16:
            raise TypeError(f"tokens must be BF16, got {tokens.dtype}")
        _require_cuda(tokens, "tokens")
        if tokens.ndim != 2 or tokens.shape[0] * repeat != n_pairs or tokens.shape[1] % 8:
            raise ValueError(f"tokens must be [{n_pairs // repeat}, width] with width % 8 == 0, got "
                             f"{tuple(tokens.shape)}")
        tok = tokens.contiguous()
        width = tok.shape[1]
        sorted_tokens = torch.empty((n_pairs, width), dtype=torch.bfloat16, device=dev)
    ad = sorted_adapters = None
    if adapter_indices is not None:
        ad = adapter_indices.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
        if ad.numel() * repeat != n_pairs:
            raise ValueError(f"adapter_indices must have {n_pairs // repeat} entries, got {ad.numel()}")
        sorted_adapters = torch.empty(n_pairs, dtype=torch.int32, device=dev)
    if out is not None:
        group_sizes, sort_indices, unsort_indices, ws = out
        if (group_sizes.numel() != num_groups or sort_indices.numel() != n_pairs or unsort_indices.numel() != n_pairs
                or ws.numel() < ws_bytes or any(t.device != dev for t in out)
                or any(t.dtype != torch.int32 for t in out[:3])):
            raise ValueError("out does not fit this dispatch")
    else:
        group_sizes = torch.empty(num_groups, dtype=torch.int32, device=dev)
        sort_indices = torch.empty(n_pairs, dtype=torch.int32, device=dev)
        unsort_indices = torch.empty(n_pairs, dtype=torch.int32, device=dev)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
    p = _native.MoeDispatchProblem()
    p.struct_size = ctypes.sizeof(_native.MoeDispatchProblem)
    p.n_pairs, p.repeat, p.width, p.n_groups = n_pairs, repeat, width, num_groups
    p.tokens = tok.data_ptr() if tok is not None else None
    p.indices = idx.data_ptr()
    p.adapter_indices = ad.data_ptr() if ad is not None else None
    p.sorted_tokens = sorted_tokens.data_ptr() if tok is not None else None
    p.group_sizes = group_sizes.data_ptr()
    p.sort_indices = sort_indices.data_ptr()
    p.unsort_indices = unsort_indices.data_ptr()
    p.sorted_adapters = sorted_adapters.data_ptr() if ad is not None else None
    p.workspace = ws.data_ptr()
    p.workspace_bytes = ws_bytes
    with torch.cuda.device(dev):
        status = lib.mi355_w8a8_moe_dispatch_v1(ctypes.byref(p), _stream_ptr(dev))
    _native.check("mi355_w8a8_moe_dispatch_v1", status)
    return sorted_tokens, group_sizes, sort_indices, unsort_indices, sorted_adapters


def prepare_routing(tokens: torch.Tensor, indices: torch.Tensor, num_groups: int,
                    adapter_indices: torch.Tensor | None = None):
    """``prepare_routing`` of skyrl/tx/layers/util.py:66-87, same arguments and results
    ``(sorted_tokens, group_sizes, unsort_indices, sorted_adapter_indices)``, on the native sort."""
    sorted_tokens, group_sizes, _, unsort, sorted_adapters = moe_dispatch(tokens, indices, num_groups,
                                                                          adapter_indices=adapter_indices)
    return sorted_tokens, group_sizes, unsort, sorted_adapters


def moe_combine(expert_out: torch.Tensor, unsort_indices: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """``sum_j expert_out[unsort[t * top_k + j]] * weights[t, j]`` in float32, one bf16 cast
    (qwen3.py:205-207).  ``expert_out`` bf16 [T * top_k, H], ``weights`` f32 [T, top_k]."""
    if expert_out.dtype != torch.bfloat16:
        raise TypeError(f"expert_out must be BF16, got {expert_out.dtype}")
    _require_cuda(expert_out, "expert_out")
    if weights.ndim != 2 or expert_out.ndim != 2 or expert_out.shape[0] != weights.numel() or expert_out.shape[1] % 8:
        raise ValueError(f"need expert_out [T * top_k, H] with H % 8 == 0 and weights [T, top_k], got "
                         f"{tuple(expert_out.shape)} and {tuple(weights.shape)}")
    if unsort_indices.numel() != weights.numel():
        raise ValueError("unsort_indices must have one entry per (token, choice)")
    dev = expert_out.device
    t, top_k = weights.shape
    eo = expert_out.contiguous()
    un = unsort_indices.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
    w = weights.detach().to(device=dev, dtype=torch.float32).contiguous()
    out = torch.empty((t, eo.shape[1]), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        status = _native.load().mi355_w8a8_moe_combine_v1(eo.data_ptr(), un.data_ptr(), w.data_ptr(), out.data_ptr(),
                                                          t, top_k, eo.shape[1], _stream_ptr(dev))
    _native.check("mi355_w8a8_moe_combine_v1", status)
    return out


def moe_combine_backward(d_out: torch.Tensor, expert_out: torch.Tensor | None, sort_indices: torch.Tensor,
                         weights: torch.Tensor, *, need_weight_grads: bool = True):
    """Pull-back of ``moe_combine``: ``d_expert_out[pos] = bf16(d_out[pair // top_k] * w[pair])`` and
    ``d_weights[pair] = <expert_out[pos], d_out[pair // top_k]>`` in float32, with
    ``pair = sort_indices[pos]`` (the derivative of qwen3.py:205-207).  Returns
    ``(d_expert_out, d_weights)``; the second is None unless asked for."""
    if d_out.dtype != torch.bfloat16:
        raise TypeError(f"d_out must be BF16, got {d_out.dtype}")
    _require_cuda(d_out, "d_out")
    if weights.ndim != 2 or d_out.ndim != 2 or d_out.shape[0] != weights.shape[0] or d_out.shape[1] % 8:
        raise ValueError(f"need d_out [T, H] with H % 8 == 0 and weights [T, top_k], got {tuple(d_out.shape)} and "
                         f"{tuple(weights.shape)}")
    t, top_k = weights.shape
    width = d_out.shape[1]
    if sort_indices.numel() != t * top_k:
        raise ValueError("sort_indices must have one entry per (token, choice)")
    dev = d_out.device
    do = d_out.contiguous()
    so = sort_indices.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
    w = weights.detach().to(device=dev, dtype=torch.float32).contiguous()
    eo = None
    if need_weight_grads:
        if expert_out is None or expert_out.dtype != torch.bfloat16 or tuple(expert_out.shape) != (t * top_k, width):
            raise ValueError(f"the weight cotangent needs expert_out BF16 [{t * top_k}, {width}]")
        eo = expert_out.contiguous()
    d_eo = torch.empty((t * top_k, width), dtype=torch.bfloat16, device=dev)
    d_w = torch.empty((t, top_k), dtype=torch.float32, device=dev) if need_weight_grads else None
    with torch.cuda.device(dev):
        status = _native.load().mi355_w8a8_moe_combine_bwd_v1(
            do.data_ptr(), eo.data_ptr() if eo is not None else None, so.data_ptr(), w.data_ptr(), d_eo.data_ptr(),
            d_w.data_ptr() if d_w is not None else None, t, top_k, width, _stream_ptr(dev))
    _native.check("mi355_w8a8_moe_combine_bwd_v1", status)
    return d_eo, d_w


class _MoeExpertMlpFunction(torch.autograd.Function):
    """The expert MLP behind the routing, differentiable in the hidden rows, the routing weights and
    the four LoRA factors: the chain of the forward written backwards (combine pull-back, grouped
    backward of the down projection, SwiGLU pull-back, grouped backward of gate/up, scatter-add of the
    gather as a combine with unit weights).  The forward keeps the gate/up projection, the activated
    rows and the down projection."""

    @staticmethod
    def forward(ctx, hidden, weights, gate_up_a, gate_up_b, down_a, down_b, lora_scaling, selected, gate_up_weight,
                down_weight, top_k):
        n_experts = gate_up_weight.n_weights
        _, group_sizes, sort_indices, unsort, _ = moe_dispatch(None, selected, n_experts, repeat=top_k)
        fused = grouped_forward(hidden, group_sizes, gate_up_weight, gate_up_a, gate_up_b, lora_scaling,
                                row_map=sort_indices, row_repeat=top_k)
        act = swiglu(fused)
        down = grouped_forward(act, group_sizes, down_weight, down_a, down_b, lora_scaling)
        ctx.save_for_backward(hidden, weights, gate_up_a, gate_up_b, down_a, down_b, lora_scaling, group_sizes,
                              sort_indices, unsort, fused, act, down)
        ctx.gate_up_weight, ctx.down_weight, ctx.top_k, ctx.selected = gate_up_weight, down_weight, top_k, selected
        return moe_combine(down, unsort, weights)

    @staticmethod
    def backward(ctx, d_out):
        (hidden, weights, gate_up_a, gate_up_b, down_a, down_b, lora_scaling, group_sizes, sort_indices, unsort, fused,
         act, down) = ctx.saved_tensors
        top_k = ctx.top_k
        lora = gate_up_a is not None
        need_lora = lora and any(ctx.needs_input_grad[2:7])
        need_w = ctx.needs_input_grad[1]
        d_down, d_w = moe_combine_backward(d_out.contiguous(), down if need_w else None, sort_indices, weights,
                                           need_weight_grads=need_w)
        d_act, d_da, d_db, ds_dn = grouped_backward(act, d_down, group_sizes, ctx.down_weight, down_a, down_b,
                                                    lora_scaling, need_lora_grads=need_lora)
        d_fused = swiglu_backward(fused, d_act)
        x_sorted = None
        if need_lora:  # the LoRA cotangents of gate/up contract over the sorted hidden rows
            x_sorted = moe_dispatch(hidden, ctx.selected, ctx.gate_up_weight.n_weights, repeat=top_k)[0]
        d_xs, d_ga, d_gb, ds_gu = grouped_backward(x_sorted, d_fused, group_sizes, ctx.gate_up_weight, gate_up_a,
                                                   gate_up_b, lora_scaling, need_lora_grads=need_lora)
        d_hidden = None
        if ctx.needs_input_grad[0]:
            d_hidden = moe_combine(d_xs, unsort, torch.ones_like(weights))
        d_s = None
        if need_lora and ctx.needs_input_grad[6]:
            d_s = ds_dn + ds_gu
            d_s = d_s.reshape(lora_scaling.shape).to(lora_scaling.dtype) if lora_scaling.ndim else d_s.sum().to(lora_scaling.dtype)
        if not need_lora:
            d_ga = d_gb = d_da = d_db = None
        return d_hidden, d_w, d_ga, d_gb, d_da, d_db, d_s, None, None, None, None


class _MoeInferencePlan:
    """The two grouped plans of an expert layer's forward without gradients, their workspaces and the
    dispatch's buffers, kept between calls with the same token count, weights and adapter tensors: the
    adapters' operand packs then survive in the workspaces (``FLAG_LORA_PACK_VALID`` while the tensors'
    ``_version`` stands), and no call allocates the intermediates anew."""

    def __init__(self, h2, top_k, gate_up_weight, down_weight, gate_up_a, gate_up_b, down_a, down_b, lora_scaling):
        dev = h2.device
        n_experts = gate_up_weight.n_weights
        n_pairs = h2.shape[0] * top_k
        lib = _native.load()
        ws_bytes = int(lib.mi355_w8a8_moe_dispatch_workspace_bytes(n_pairs, n_experts))
        if ws_bytes == 0:
            raise ValueError(f"{n_pairs} rows in {n_experts} groups are outside the native dispatch")
        self.dispatch_out = (torch.zeros(n_experts, dtype=torch.int32, device=dev),
                             torch.zeros(n_pairs, dtype=torch.int32, device=dev),
                             torch.zeros(n_pairs, dtype=torch.int32, device=dev),
                             torch.empty(ws_bytes, dtype=torch.uint8, device=dev))
        sizes, sort_indices, _, _ = self.dispatch_out
        self.gate_up = GroupedForwardPlan(h2, sizes, gate_up_weight, gate_up_a, gate_up_b, lora_scaling, swiglu=True,
                                          row_map=sort_indices, row_repeat=top_k)
        self.down = GroupedForwardPlan(self.gate_up.out, sizes, down_weight, down_a, down_b, lora_scaling)
        # the plans must read the dispatch's own buffers, not converted copies
        assert self.gate_up.group_sizes.data_ptr() == sizes.data_ptr() == self.down.group_sizes.data_ptr()
        assert self.gate_up.row_map.data_ptr() == sort_indices.data_ptr()
        self.top_k, self.n_experts = top_k, n_experts
        refs = [t for t in (gate_up_a, gate_up_b, down_a, down_b) if t is not None]
        self._lora_refs = [weakref.ref(t) for t in refs]
        self._down_weight = weakref.ref(down_weight)
        self._scaling = lora_scaling if not isinstance(lora_scaling, torch.Tensor) else (weakref.ref(lora_scaling),
                                                                                          _version_of(lora_scaling))
        self._shape = (tuple(h2.shape), h2.device)

    def fits(self, h2, top_k, down_weight, lora, lora_scaling) -> bool:
        if self._shape != (tuple(h2.shape), h2.device) or self.top_k != top_k or self._down_weight() is not down_weight:
            return False
        given = [t for t in lora if t is not None]
        if len(given) != len(self._lora_refs) or any(r() is not t for r, t in zip(self._lora_refs, given)):
            return False
        if isinstance(lora_scaling, torch.Tensor):
            return (isinstance(self._scaling, tuple) and self._scaling[0]() is lora_scaling
                    and self._scaling[1] is not None and self._scaling[1] == _version_of(lora_scaling))
        return not isinstance(self._scaling, tuple) and self._scaling == lora_scaling

    def run(self, h2, selected, weights):
        _, _, _, unsort, _ = moe_dispatch(None, selected, self.n_experts, repeat=self.top_k, out=self.dispatch_out)
        self.gate_up.bind_x(h2)
        self.gate_up.run()
        down = self.down.run()
        return moe_combine(down, unsort, weights)


_moe_inference_plans = weakref.WeakKeyDictionary()  # gate/up weight -> the layer's plan (one token count at a time)


def moe_expert_mlp(hidden, router_logits, top_k: int, gate_up_weight, down_weight, gate_up_a=None, gate_up_b=None,
                   down_a=None, down_b=None, lora_scaling=None, *, norm_topk_prob: bool = True):
    """Expert MLP of ``Qwen3Experts.__call__`` (skyrl/tx/models/qwen3.py:172-210) on W8A8 weights.
    Without gradients: five native calls (route, dispatch of indices, grouped gate/up + SwiGLU reading
    the hidden rows through the sort order, grouped down, combine).  Under autograd the same values
    come from the projection without the fused SwiGLU plus the stand-alone SwiGLU kernel, and the call
    is differentiable in ``hidden``, ``router_logits`` (through the routing weights, the selection
    held fixed as ``lax.top_k`` does) and the LoRA factors and scaling."""
    n_experts = gate_up_weight.n_weights
    h2 = hidden.reshape(-1, hidden.shape[-1])
    tensors = [t for t in (hidden, router_logits, gate_up_a, gate_up_b, down_a, down_b, lora_scaling)
               if isinstance(t, torch.Tensor)]
    training = torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    logits2 = router_logits.reshape(-1, router_logits.shape[-1])
    if training and router_logits.requires_grad:
        weights, selected = _MoeRouteFunction.apply(logits2, top_k, norm_topk_prob)
    else:
        weights, selected = moe_route(logits2, top_k, norm_topk_prob)
    if not training:
        # indices only: the first projection gathers the hidden rows itself through the sort order.  The
        # layer's plans are kept with its gate/up weight: calls that share a weight object must be ordered on
        # one stream (they share the intermediates), and not captured into different graphs.
        h2 = h2.contiguous()
        plan = _moe_inference_plans.get(gate_up_weight)
        if plan is None or not plan.fits(h2, top_k, down_weight, (gate_up_a, gate_up_b, down_a, down_b), lora_scaling):
            plan = _MoeInferencePlan(h2, top_k, gate_up_weight, down_weight, gate_up_a, gate_up_b, down_a, down_b,
                                     lora_scaling)
            _moe_inference_plans[gate_up_weight] = plan
        return plan.run(h2, selected, weights).reshape(hidden.shape)
    scaling = lora_scaling
    if gate_up_a is not None and not isinstance(scaling, torch.Tensor):
        scaling = _scaling_scalar(scaling, hidden.device)
    out = _MoeExpertMlpFunction.apply(h2, weights, gate_up_a, gate_up_b, down_a, down_b, scaling, selected,
                                      gate_up_weight, down_weight, top_k)
    return out.reshape(hidden.shape)


def w8a8_moe_expert_mlp(hidden, router_logits, top_k: int, gate_up_weight, down_weight, gate_up_a, gate_up_b,
                        down_a, down_b, lora_scaling, *, enabled: bool = False, norm_topk_prob: bool = True):
    """``moe_expert_mlp`` behind the reference's opt-in switch."""
    _check_enabled(enabled, False, "MoE expert MLP")
    return moe_expert_mlp(hidden, router_logits, top_k, gate_up_weight, down_weight, gate_up_a, gate_up_b, down_a,
                          down_b, lora_scaling, norm_topk_prob=norm_topk_prob)


def _check_enabled(enabled, interpret, what: str) -> None:
    _validate_exact_bool("enabled", enabled)
    _validate_exact_bool("interpret", interpret)
    if not enabled:
        raise RuntimeError(f"the W8A8 {what} path is disabled by default")
    if interpret:
        raise RuntimeError("interpret=True is not available: the HIP build has no interpreter or CPU path")


def _check_tiles(block_m, block_n, row_superblock) -> None:
    _validate_block_size("block_m", block_m, MAX_BLOCK_M)
    _validate_block_size("block_n", block_n, MAX_BLOCK_N)
    _validate_row_superblock(row_superblock, block_m)


def w8a8_frozen_linear(x, weight, *, enabled: bool = False, interpret: bool = False,
                       block_m: int = DEFAULT_BLOCK_M, block_n: int = DEFAULT_BLOCK_N,
                       row_superblock: int = DEFAULT_ROW_SUPERBLOCK):
    """Frozen W8A8 base only: bf16(dequant(quant(x) @ Wq))."""
    _check_enabled(enabled, interpret, "frozen-linear")
    _check_tiles(block_m, block_n, row_superblock)
    return lora_linear(x, weight)


def w8a8_lora_linear(x, weight, lora_a, lora_b, lora_scaling, *, enabled: bool = False,
                     interpret: bool = False, block_m: int = DEFAULT_BLOCK_M,
                     block_n: int = DEFAULT_BLOCK_N, row_superblock: int = DEFAULT_ROW_SUPERBLOCK,
                     adapter_indices=None):
    """Frozen W8A8 base + LoRA in one float32 epilogue and one bf16 cast.

    ``lora_a``/``lora_b`` are [K, r]/[r, N] with a scalar ``lora_scaling``, or stacked
    [n, K, r]/[n, r, N] with ``lora_scaling`` [n] and ``adapter_indices`` selecting
    an adapter per row (or per example).
    """
    _check_enabled(enabled, interpret, "LoRA")
    _check_tiles(block_m, block_n, row_superblock)
    if lora_a.ndim == 2:
        scaling = torch.as_tensor(lora_scaling, dtype=torch.float32)
        if scaling.ndim != 0:
            raise TypeError("lora_scaling must be an FP32 scalar")
    return lora_linear(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices)


def w8a8_rms_gate_up_lora_swiglu(x, rms_weight, weight, lora_a, lora_b, lora_scaling, *,
                                 enabled: bool = False, eps: float = 1e-6, interpret: bool = False,
                                 rms_is_delta: bool = False, adapter_indices=None):
    """RMSNorm -> W8A8 gate/up (+LoRA) -> SwiGLU; fused columns are (gate, up) interleaved.

    ``rms_weight`` multiplies the normalized rows (Qwen3); with ``rms_is_delta`` it is
    the Qwen3.5 delta and the multiplier is ``1 + delta`` evaluated in float32.  Differentiable in
    x and the LoRA parameters; the norm weight and the frozen kernel are constants.
    """
    _check_enabled(enabled, interpret, "RMSNorm gate/up SwiGLU")
    _validate_exact_bool("rms_is_delta", rms_is_delta)
    gamma = rms_weight.detach().to(torch.float32)
    if rms_is_delta:
        gamma = 1.0 + gamma
    return rms_gate_up_lora_swiglu(x, gamma, weight, lora_a, lora_b, lora_scaling,
                                   adapter_indices=adapter_indices, eps=eps)


def w8a8_lora_residual(x, weight, lora_a, lora_b, lora_scaling, residual, *, enabled: bool = False,
                       interpret: bool = False, adapter_indices=None):
    """W8A8 down projection + LoRA + residual, summed in float32 and cast once."""
    _check_enabled(enabled, interpret, "LoRA residual")
    if residual is None:
        raise ValueError("w8a8_lora_residual needs a residual")
    return lora_linear(x, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices, residual=residual)


# ---------------------------------------------------------------------------------------
# Qwen3.5 attention input stage (skyrl/tx/kernels/qwen3_5_qkv_lora.py)
# ---------------------------------------------------------------------------------------
@dataclass(frozen=True)
class Qwen35QKVStageConfig:
    """Static geometry of the stage (qwen3_5_qkv_lora.py:36-85, same fields and checks)."""

    num_query_heads: int
    num_kv_heads: int
    head_dim: int
    rotary_dim: int
    rope_theta: float
    rms_norm_eps: float

    def __post_init__(self) -> None:
        if self.num_query_heads <= 0 or self.num_kv_heads <= 0:
            raise ValueError("num_query_heads and num_kv_heads must be positive")
        if self.num_query_heads % self.num_kv_heads != 0:
            raise ValueError("num_query_heads must be divisible by num_kv_heads")
        if self.head_dim <= 0:
            raise ValueError("head_dim must be positive")
        if self.rotary_dim < 0 or self.rotary_dim > self.head_dim or self.rotary_dim % 2:
            raise ValueError("rotary_dim must be even and lie in [0, head_dim]")
        if self.rope_theta <= 0:
            raise ValueError("rope_theta must be positive")
        if self.rms_norm_eps <= 0:
            raise ValueError("rms_norm_eps must be positive")

    @property
    def queries_per_kv(self) -> int:
        return self.num_query_heads // self.num_kv_heads

    @property
    def q_projection_width(self) -> int:
        return self.num_query_heads * 2 * self.head_dim

    @property
    def kv_projection_width(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def fused_width(self) -> int:
        return self.q_projection_width + 2 * self.kv_projection_width


class QkvPostPlan:
    """Outputs and the C struct of one split / Q-K norm / partial-RoPE call; ``run()`` is a single
    C call on torch's current stream (see ``ForwardPlan``)."""

    def __init__(self, fused: torch.Tensor, q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor,
                 positions: torch.Tensor, config: Qwen35QKVStageConfig):
        if fused.dtype != torch.bfloat16:
            raise TypeError(f"fused must be BF16, got {fused.dtype}")
        _require_cuda(fused, "fused")
        if fused.shape[-1] != config.fused_width:
            raise ValueError(f"fused width {fused.shape[-1]} does not match the configuration ({config.fused_width})")
        lead = tuple(fused.shape[:-1])
        if tuple(positions.shape) != lead:
            raise ValueError(f"positions must have shape {lead}, got {tuple(positions.shape)}")
        d = config.head_dim
        if tuple(q_norm_weight.shape) != (d,) or tuple(k_norm_weight.shape) != (d,):
            raise ValueError(f"q_norm_weight and k_norm_weight must have shape ({d},)")
        dev = fused.device
        flat = fused.reshape(-1, config.fused_width).contiguous()
        m = flat.shape[0]
        qw = q_norm_weight.to(device=dev, dtype=torch.float32).contiguous()
        kw = k_norm_weight.to(device=dev, dtype=torch.float32).contiguous()
        pos = positions.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
        self.q = torch.empty((m, config.num_query_heads, d), dtype=torch.bfloat16, device=dev)
        self.k = torch.empty((m, config.num_kv_heads, d), dtype=torch.bfloat16, device=dev)
        self.v = torch.empty((m, config.num_kv_heads, d), dtype=torch.bfloat16, device=dev)
        self.gate = torch.empty((m, config.num_query_heads * d), dtype=torch.bfloat16, device=dev)
        p = _native.QkvPostProblem()
        p.struct_size = ctypes.sizeof(_native.QkvPostProblem)
        p.m, p.num_query_heads, p.num_kv_heads = m, config.num_query_heads, config.num_kv_heads
        p.head_dim, p.rotary_dim = d, config.rotary_dim
        p.rope_theta, p.rms_eps = float(config.rope_theta), float(config.rms_norm_eps)
        p.fused, p.q_norm_weight, p.k_norm_weight = flat.data_ptr(), qw.data_ptr(), kw.data_ptr()
        p.positions = pos.data_ptr()
        p.q, p.k, p.v, p.gate = self.q.data_ptr(), self.k.data_ptr(), self.v.data_ptr(), self.gate.data_ptr()
        self.problem = p
        self.device = dev
        self.lead = lead
        self.config = config
        self._fn = _native.load().mi355_w8a8_qkv_split_norm_rope_v1
        self._keep = (flat, qw, kw, pos)

    def run(self):
        with torch.cuda.device(self.device):
            status = self._fn(ctypes.byref(self.problem), _stream_ptr(self.device))
        _native.check("mi355_w8a8_qkv_split_norm_rope_v1", status)
        c, lead = self.config, self.lead
        return (self.q.reshape(*lead, c.num_query_heads, c.head_dim), self.k.reshape(*lead, c.num_kv_heads, c.head_dim),
                self.v.reshape(*lead, c.num_kv_heads, c.head_dim), self.gate.reshape(*lead, c.num_query_heads * c.head_dim))


def qkv_split_norm_rope(fused: torch.Tensor, q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor,
                        positions: torch.Tensor, config: Qwen35QKVStageConfig):
    """Split of the interleaved projection, Q/K RMSNorm with ``1 + weight``, partial RoPE
    (qwen3_5_qkv_lora.py:266-286).  ``fused`` is bf16 [..., fused_width], ``positions`` int [...].
    Returns q [..., Hq, D], k [..., Hkv, D], v [..., Hkv, D], gate [..., Hq * D]."""
    return QkvPostPlan(fused, q_norm_weight, k_norm_weight, positions, config).run()


def qkv_split_norm_rope_backward(fused: torch.Tensor, q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor,
                                 positions: torch.Tensor, config: Qwen35QKVStageConfig, d_q, d_k, d_v, d_gate, *,
                                 need_norm_weight_grads: bool = False):
    """Pull-back of ``qkv_split_norm_rope`` (qwen3_5_qkv_lora.py:391-425): ``fused`` is the raw bf16
    projection the forward consumed; a missing output cotangent (None) counts as zero.  Returns
    ``(d_fused, d_q_norm_weight, d_k_norm_weight)``, the last two float32 [head_dim] or None."""
    if fused.dtype != torch.bfloat16:
        raise TypeError(f"fused must be BF16, got {fused.dtype}")
    _require_cuda(fused, "fused")
    if fused.shape[-1] != config.fused_width:
        raise ValueError(f"fused width {fused.shape[-1]} does not match the configuration ({config.fused_width})")
    lead = tuple(fused.shape[:-1])
    if tuple(positions.shape) != lead:
        raise ValueError(f"positions must have shape {lead}, got {tuple(positions.shape)}")
    d, hq, hkv = config.head_dim, config.num_query_heads, config.num_kv_heads
    if tuple(q_norm_weight.shape) != (d,) or tuple(k_norm_weight.shape) != (d,):
        raise ValueError(f"q_norm_weight and k_norm_weight must have shape ({d},)")
    dev = fused.device
    flat = fused.reshape(-1, config.fused_width).contiguous()
    m = flat.shape[0]

    def cot(t, width, name):
        if t is None:
            return torch.zeros((m, width), dtype=torch.bfloat16, device=dev)
        if t.dtype != torch.bfloat16:
            raise TypeError(f"{name} must be BF16, got {t.dtype}")
        if t.numel() != m * width:
            raise ValueError(f"{name} must hold {m} x {width} elements, got {tuple(t.shape)}")
        return t.reshape(m, width).contiguous()

    dq, dk = cot(d_q, hq * d, "d_q"), cot(d_k, hkv * d, "d_k")
    dv, dg = cot(d_v, hkv * d, "d_v"), cot(d_gate, hq * d, "d_gate")
    qw = q_norm_weight.to(device=dev, dtype=torch.float32).contiguous()
    kw = k_norm_weight.to(device=dev, dtype=torch.float32).contiguous()
    pos = positions.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
    d_fused = torch.empty_like(flat)
    lib = _native.load()
    p = _native.QkvPostBwdProblem()
    p.struct_size = ctypes.sizeof(_native.QkvPostBwdProblem)
    p.m, p.num_query_heads, p.num_kv_heads, p.head_dim, p.rotary_dim = m, hq, hkv, d, config.rotary_dim
    p.rope_theta, p.rms_eps = float(config.rope_theta), float(config.rms_norm_eps)
    p.fused, p.q_norm_weight, p.k_norm_weight, p.positions = flat.data_ptr(), qw.data_ptr(), kw.data_ptr(), pos.data_ptr()
    p.d_q, p.d_k, p.d_v, p.d_gate, p.d_fused = dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dg.data_ptr(), d_fused.data_ptr()
    dqw = dkw = ws = None
    if need_norm_weight_grads:
        dqw = torch.empty(d, dtype=torch.float32, device=dev)
        dkw = torch.empty(d, dtype=torch.float32, device=dev)
        ws = torch.empty(int(lib.mi355_w8a8_qkv_bwd_workspace_bytes(m, d)), dtype=torch.uint8, device=dev)
        p.d_q_norm_weight, p.d_k_norm_weight = dqw.data_ptr(), dkw.data_ptr()
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
    with torch.cuda.device(dev):
        status = lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1(ctypes.byref(p), _stream_ptr(dev))
    _native.check("mi355_w8a8_qkv_split_norm_rope_bwd_v1", status)
    return d_fused.reshape(fused.shape), dqw, dkw


def delta_rms_norm_backward(x: torch.Tensor, gamma: torch.Tensor, d_normalized: torch.Tensor, *, eps: float = 1e-6,
                            need_weight_grad: bool = False, in_place: bool = False):
    """Pull-back of ``bf16(x * rsqrt(mean(x^2) + eps) * gamma)`` in the form of ``_delta_rms_norm_vjp``
    (qwen3_5_qkv_lora.py:97-116); ``gamma`` float32 [K] is the multiplier ``1 + weight``.  Returns
    ``(d_x, d_weight)``; ``d_weight`` float32 [K] (None unless asked for) is the cotangent of the
    weight.  ``in_place`` overwrites ``d_normalized`` and excludes ``need_weight_grad``."""
    if x.dtype != torch.bfloat16 or d_normalized.dtype != torch.bfloat16:
        raise TypeError("x and d_normalized must be BF16")
    _require_cuda(x, "x")
    _require_cuda(d_normalized, "d_normalized")
    k = x.shape[-1]
    if x.ndim < 2 or tuple(d_normalized.shape) != tuple(x.shape) or tuple(gamma.shape) != (k,):
        raise ValueError(f"need x and d_normalized [..., K] and gamma [K], got {tuple(x.shape)}, "
                         f"{tuple(d_normalized.shape)} and {tuple(gamma.shape)}")
    if not isinstance(eps, float) or not eps > 0.0:
        raise ValueError(f"eps must be a positive float, got {eps!r}")
    if in_place and need_weight_grad:
        raise ValueError("the weight cotangent reads d_normalized after d_x is written: not in place")
    if in_place and not d_normalized.is_contiguous():
        raise ValueError("in_place needs a contiguous d_normalized tensor")
    x2 = x.reshape(-1, k).contiguous()
    d2 = d_normalized.reshape(-1, k).contiguous()
    g = gamma.to(device=x.device, dtype=torch.float32).contiguous()
    out = d2 if in_place else torch.empty_like(d2)
    lib = _native.load()
    dw = ws = None
    dw_ptr = ws_ptr = ws_bytes = 0
    if need_weight_grad:
        dw = torch.empty(k, dtype=torch.float32, device=x.device)
        ws = torch.empty(int(lib.mi355_w8a8_delta_rms_norm_bwd_workspace_bytes(x2.shape[0], k)), dtype=torch.uint8,
                         device=x.device)
        dw_ptr, ws_ptr, ws_bytes = dw.data_ptr(), ws.data_ptr(), ws.numel()
    with torch.cuda.device(x.device):
        status = lib.mi355_w8a8_delta_rms_norm_bwd_v1(x2.data_ptr(), g.data_ptr(), d2.data_ptr(), out.data_ptr(), dw_ptr,
                                                      ws_ptr, ws_bytes, x2.shape[0], k, eps, _stream_ptr(x.device))
    _native.check("mi355_w8a8_delta_rms_norm_bwd_v1", status)
    return out.reshape(x.shape), dw


class QkvStageBackwardPlan:
    """Buffers and C structs of one backward of the attention input stage with frozen norm weights
    (the LoRA-training case): ``run()`` enqueues the forward recomputation (unless the projection and
    the normalized rows are handed in), the split / norm / RoPE pull-back, the linear backward and the
    decoder-norm pull-back in place on that call's dx.  Repeated calls reuse every buffer."""

    def __init__(self, hidden: torch.Tensor, input_norm_weight: torch.Tensor, q_norm_weight: torch.Tensor,
                 k_norm_weight: torch.Tensor, weight, lora_a, lora_b, lora_scaling, positions: torch.Tensor,
                 config: Qwen35QKVStageConfig, d_q, d_k, d_v, d_gate, *, adapter_indices=None,
                 need_lora_grads: bool = True, fused: torch.Tensor | None = None,
                 normalized: torch.Tensor | None = None):
        if (fused is None) != (normalized is None):
            raise ValueError("hand in both the projection and the normalized rows, or neither")
        dev = hidden.device
        d, hq, hkv = config.head_dim, config.num_query_heads, config.num_kv_heads
        k = hidden.shape[-1]
        gamma = (1.0 + input_norm_weight.detach().to(torch.float32)).to(dev).contiguous()
        self.fwd = None
        if fused is None:
            self.fwd = ForwardPlan(hidden, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                                   rms_gamma=gamma, eps=config.rms_norm_eps, want_normalized=True)
            fused, normalized = self.fwd.out, self.fwd.aux["normalized"]
        if fused.dtype != torch.bfloat16 or fused.shape[-1] != config.fused_width:
            raise ValueError("fused must be the bf16 projection of this configuration")
        flat = fused.reshape(-1, config.fused_width).contiguous()
        m = flat.shape[0]
        if hidden.numel() != m * k or normalized.numel() != m * k:
            raise ValueError("hidden, normalized and fused disagree on the number of rows")

        def cot(t, width, name):
            if t is None:
                return torch.zeros((m, width), dtype=torch.bfloat16, device=dev)
            if t.dtype != torch.bfloat16 or t.numel() != m * width:
                raise ValueError(f"{name} must be BF16 with {m} x {width} elements")
            return t.reshape(m, width).contiguous()

        cots = (cot(d_q, hq * d, "d_q"), cot(d_k, hkv * d, "d_k"), cot(d_v, hkv * d, "d_v"), cot(d_gate, hq * d, "d_gate"))
        qw = q_norm_weight.detach().to(device=dev, dtype=torch.float32).contiguous()
        kw = k_norm_weight.detach().to(device=dev, dtype=torch.float32).contiguous()
        pos = positions.reshape(-1).to(device=dev, dtype=torch.int32).contiguous()
        if pos.numel() != m:
            raise ValueError(f"positions must name {m} rows, got {tuple(positions.shape)}")
        self.d_fused = torch.empty_like(flat)
        p = _native.QkvPostBwdProblem()
        p.struct_size = ctypes.sizeof(_native.QkvPostBwdProblem)
        p.m, p.num_query_heads, p.num_kv_heads, p.head_dim, p.rotary_dim = m, hq, hkv, d, config.rotary_dim
        p.rope_theta, p.rms_eps = float(config.rope_theta), float(config.rms_norm_eps)
        p.fused, p.q_norm_weight, p.k_norm_weight, p.positions = flat.data_ptr(), qw.data_ptr(), kw.data_ptr(), pos.data_ptr()
        p.d_q, p.d_k, p.d_v, p.d_gate = (c.data_ptr() for c in cots)
        p.d_fused = self.d_fused.data_ptr()
        self.post_problem = p
        idx = adapter_indices
        if idx is not None and idx.numel() != m:
            idx = idx.reshape(-1).repeat_interleave(m // idx.numel())
        self.bwd = BackwardPlan(normalized.reshape(m, k), self.d_fused, weight, lora_a, lora_b, lora_scaling,
                                adapter_indices=idx, need_lora_grads=need_lora_grads)
        self.x = hidden.reshape(m, k).contiguous()
        self.gamma, self.eps = gamma, float(config.rms_norm_eps)
        self.device, self.dx_shape, self.m, self.k = dev, tuple(hidden.shape), m, k
        self._lib = _native.load()
        self._keep = (flat, normalized, cots, qw, kw, pos)

    def run_post_stage(self) -> None:
        with torch.cuda.device(self.device):
            status = self._lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1(ctypes.byref(self.post_problem),
                                                                     _stream_ptr(self.device))
        _native.check("mi355_w8a8_qkv_split_norm_rope_bwd_v1", status)

    def run_rms_stage(self) -> None:
        dx = self.bwd.dx
        with torch.cuda.device(self.device):
            status = self._lib.mi355_w8a8_delta_rms_norm_bwd_v1(self.x.data_ptr(), self.gamma.data_ptr(), dx.data_ptr(),
                                                                dx.data_ptr(), None, None, 0, self.m, self.k, self.eps,
                                                                _stream_ptr(self.device))
        _native.check("mi355_w8a8_delta_rms_norm_bwd_v1", status)

    def run(self):
        """Returns ``(d_hidden, d_lora_a, d_lora_b, d_lora_scaling)`` (reused tensors)."""
        if self.fwd is not None:
            self.fwd.run()
        self.run_post_stage()
        dn, da, db, ds = self.bwd.run()
        self.run_rms_stage()
        return dn.reshape(self.dx_shape), da, db, ds


class _QkvStageFunction(torch.autograd.Function):
    """The stage with the derivative rule of ``_qwen35_qkv_lora_rope`` (qwen3_5_qkv_lora.py:288-454):
    cotangents for the hidden rows, the three norm weights, A, B and the scaling; none for the frozen
    kernel and the positions.  The forward keeps the bf16 projection and the normalized rows
    (``save_projection``) or nothing beyond its inputs, in which case the backward recomputes both
    with one forward call, as the reference's rule does (:378-388)."""

    @staticmethod
    def forward(ctx, hidden, input_norm_weight, q_norm_weight, k_norm_weight, lora_a, lora_b, lora_scaling, weight,
                positions, config, adapter_indices, save_projection):
        ctx.weight, ctx.config, ctx.adapter_indices = weight, config, adapter_indices
        ctx.saved_projection = bool(save_projection)
        gamma = 1.0 + input_norm_weight.detach().to(torch.float32)
        plan = ForwardPlan(hidden, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                           rms_gamma=gamma, eps=config.rms_norm_eps, want_normalized=ctx.saved_projection)
        fused = plan.run()
        keep = (fused, plan.aux["normalized"]) if ctx.saved_projection else ()
        ctx.save_for_backward(hidden, input_norm_weight, q_norm_weight, k_norm_weight, lora_a, lora_b, lora_scaling,
                              positions, *keep)
        q, k, v, gate = qkv_split_norm_rope(fused, q_norm_weight, k_norm_weight, positions, config)
        return q, k, v, gate

    @staticmethod
    def backward(ctx, d_q, d_k, d_v, d_gate):
        hidden, in_w, q_w, k_w, lora_a, lora_b, lora_scaling, positions = ctx.saved_tensors[:8]
        config = ctx.config
        gamma = 1.0 + in_w.detach().to(torch.float32)
        if ctx.saved_projection:
            fused, normalized = ctx.saved_tensors[8:]
        else:
            plan = ForwardPlan(hidden, ctx.weight, lora_a, lora_b, lora_scaling, adapter_indices=ctx.adapter_indices,
                               rms_gamma=gamma, eps=config.rms_norm_eps, want_normalized=True)
            fused = plan.run()
            normalized = plan.aux["normalized"]
        need_lora = lora_a is not None and any(ctx.needs_input_grad[4:7])
        need_head = ctx.needs_input_grad[2] or ctx.needs_input_grad[3]
        need_in = ctx.needs_input_grad[1]
        d_fused, dqw, dkw = qkv_split_norm_rope_backward(fused, q_w, k_w, positions, config, d_q, d_k, d_v, d_gate,
                                                         need_norm_weight_grads=need_head)
        rows = normalized.shape[0]
        idx = ctx.adapter_indices
        if idx is not None and idx.numel() != rows:
            idx = idx.reshape(-1).repeat_interleave(rows // idx.numel())
        dn, da, db, ds = backward(normalized, d_fused.reshape(rows, -1), ctx.weight, lora_a, lora_b, lora_scaling,
                                  adapter_indices=idx, need_lora_grads=need_lora)
        dh, dinw = delta_rms_norm_backward(hidden.reshape(rows, -1), gamma, dn, eps=config.rms_norm_eps,
                                           need_weight_grad=need_in, in_place=not need_in)
        if need_lora:
            if lora_a.ndim == 2:
                da, db = da[0], db[0]
            ds = ds.reshape(lora_scaling.shape).to(lora_scaling.dtype)
        else:
            da = db = ds = None
        dinw = dinw.to(in_w.dtype) if need_in else None
        dqw = dqw.to(q_w.dtype) if ctx.needs_input_grad[2] else None
        dkw = dkw.to(k_w.dtype) if ctx.needs_input_grad[3] else None
        return dh.reshape(hidden.shape), dinw, dqw, dkw, da, db, ds, None, None, None, None, None


def qkv_lora_rope(hidden, input_norm_weight, q_norm_weight, k_norm_weight, weight, lora_a, lora_b, lora_scaling,
                  positions, *, config: Qwen35QKVStageConfig, adapter_indices=None, save_projection: bool = True):
    """The attention input stage that autograd can differentiate in the hidden rows, the norm weights
    and the LoRA parameters.  ``save_projection`` keeps 2 * M * (fused width + K) bytes until the
    backward instead of recomputing the projection there."""
    tensors = [t for t in (hidden, input_norm_weight, q_norm_weight, k_norm_weight, lora_a, lora_b, lora_scaling)
               if isinstance(t, torch.Tensor)]
    if not (torch.is_grad_enabled() and any(t.requires_grad for t in tensors)):
        gamma = 1.0 + input_norm_weight.to(torch.float32)
        fused = forward(hidden, weight, lora_a, lora_b, lora_scaling, adapter_indices=adapter_indices,
                        rms_gamma=gamma, eps=config.rms_norm_eps)
        return qkv_split_norm_rope(fused, q_norm_weight, k_norm_weight, positions, config)
    scaling = lora_scaling
    if lora_a is not None and not isinstance(scaling, torch.Tensor):
        scaling = _scaling_scalar(scaling, hidden.device)
    return _QkvStageFunction.apply(hidden, input_norm_weight, q_norm_weight, k_norm_weight, lora_a, lora_b, scaling,
                                   weight, positions, config, adapter_indices, save_projection)


def w8a8_qkv_lora_rope(hidden, input_norm_weight, q_norm_weight, k_norm_weight, weight, lora_a, lora_b, lora_scaling,
                       positions, *, config: Qwen35QKVStageConfig, adapter_indices=None, enabled: bool = False,
                       interpret: bool = False, save_projection: bool = True):
    """``qwen35_qkv_lora_rope`` (qwen3_5_qkv_lora.py:532-…) with the W8A8 projection in the place of
    the bf16 one: decoder RMSNorm (delta weights) fused into the quantizer, W8A8 QKV + LoRA in one
    float32 epilogue, then the split / Q-K norm / partial-RoPE kernel; under autograd with the
    derivative rule of ``_qwen35_qkv_lora_rope_bwd`` (:360-451)."""
    _check_enabled(enabled, interpret, "QKV input stage")
    return qkv_lora_rope(hidden, input_norm_weight, q_norm_weight, k_norm_weight, weight, lora_a, lora_b,
                         lora_scaling, positions, config=config, adapter_indices=adapter_indices,
                         save_projection=save_projection)


__all__ = (
    "DEFAULT_BLOCK_M", "DEFAULT_BLOCK_N", "DEFAULT_ROW_SUPERBLOCK", "MAX_BLOCK_M", "MAX_BLOCK_N",
    "MAX_IN_FEATURES", "MAX_OUT_FEATURES", "MAX_ROW_SUPERBLOCK", "MAX_LORA_RANK", "PackedW8Weight",
    "prepare_weight", "unpack_weight", "dynamic_quantize_rows", "ForwardPlan", "forward", "BackwardPlan", "backward", "lora_linear",
    "w8a8_frozen_linear",
    "w8a8_lora_linear", "w8a8_rms_gate_up_lora_swiglu", "w8a8_lora_residual", "PackedGroupedW8Weight",
    "prepare_grouped_weight", "grouped_forward", "grouped_backward", "grouped_backward_per_weight",
    "GroupedBackwardPlan", "GroupedForwardPlan", "grouped_lora_linear",
    "w8a8_grouped_lora_linear", "w8a8_moe_expert_mlp", "moe_expert_mlp", "moe_combine_backward", "moe_route_backward", "Qwen35QKVStageConfig", "QkvPostPlan", "qkv_split_norm_rope",
    "w8a8_qkv_lora_rope", "qkv_lora_rope", "qkv_split_norm_rope_backward", "delta_rms_norm_backward", "QkvStageBackwardPlan",
)
