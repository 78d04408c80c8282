"""ctypes binding of ``libmi355_w8a8.so`` (the C ABI declared in include/mi355_w8a8.h).

The library is loaded from ``lib/`` next to this file.  There is no CPU fallback: if
the library is missing, or a launch is refused, the caller gets an exception.
"""

from __future__ import annotations

import ctypes
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libmi355_w8a8.so"

ABI_VERSION = 1
FLAG_SWIGLU = 1
FLAG_FORCE_TILED = 2
FLAG_FORCE_SKINNY = 4
FLAG_LORA_SPLIT2 = 8
FLAG_SKIP_PROLOGUE = 16
FLAG_SKIP_GEMM = 32
FLAG_TILE_256X128 = 64
FLAG_TILE_256X256 = 128
FLAG_GROUPED_TILE64 = 256
FLAG_GROUPED_TILE128 = 512
FLAG_LORA_PACK_VALID = 1024
FLAG_TILE_128X128 = 2048
FLAG_TILE_256X128_PAIR = 4096
FLAG_GQ_DIRECT = 1  # mi355_w8a8_gq_problem.flags
STATIC_WORKSPACE_BYTES = 32 << 20
PATH_NAMES = {1: "skinny", 2: "skinny-chunks", 3: "tiled-256x128", 4: "tiled-256x256", 5: "tiled-128x128",
              6: "tiled-256x128-pair"}

STATUS = {
    0: "OK", -1: "ERR_NULL", -2: "ERR_SHAPE", -3: "ERR_ALIGN", -4: "ERR_ALIAS",
    -5: "ERR_WORKSPACE", -6: "ERR_LAUNCH", -7: "ERR_UNSUPPORTED", -8: "ERR_STRUCT",
}

EXPORTS = (
    "mi355_w8a8_abi_version", "mi355_w8a8_status_string", "mi355_w8a8_packed_weight_bytes",
    "mi355_w8a8_pack_weight_v1", "mi355_w8a8_unpack_weight_v1", "mi355_w8a8_quantize_rows_v1",
    "mi355_w8a8_workspace_bytes", "mi355_w8a8_grouped_workspace_bytes",
    "mi355_w8a8_lora_linear_v1", "mi355_w8a8_rms_gateup_swiglu_v1", "mi355_w8a8_lora_residual_v1",
    "mi355_w8a8_forward_v1", "mi355_w8a8_forward_static_ws_v1", "mi355_w8a8_grouped_v1",
    "mi355_w8a8_bwd_workspace_bytes", "mi355_w8a8_lora_linear_bwd_v1",
    "mi355_w8a8_grouped_bwd_workspace_bytes", "mi355_w8a8_grouped_bwd_v1",
    "mi355_w8a8_qkv_split_norm_rope_v1",
    "mi355_w8a8_qkv_bwd_workspace_bytes", "mi355_w8a8_qkv_split_norm_rope_bwd_v1",
    "mi355_w8a8_delta_rms_norm_bwd_workspace_bytes", "mi355_w8a8_delta_rms_norm_bwd_v1",
    "mi355_w8a8_swiglu_v1", "mi355_w8a8_swiglu_bwd_v1", "mi355_w8a8_rms_norm_bwd_v1",
    "mi355_w8a8_moe_route_v1", "mi355_w8a8_moe_route_bwd_v1", "mi355_w8a8_moe_dispatch_workspace_bytes", "mi355_w8a8_moe_dispatch_v1",
    "mi355_w8a8_moe_combine_v1", "mi355_w8a8_moe_combine_bwd_v1",
    "mi355_w8a8_gq_packed_weight_bytes", "mi355_w8a8_gq_pack_weight_v1", "mi355_w8a8_gq_workspace_bytes",
    "mi355_w8a8_gq_linear_v1",
    "mi355_w8a8_forward_path", "mi355_w8a8_calibrate_operand_bytes", "mi355_w8a8_calibrate_mfma_ops", "mi355_w8a8_calibrate_mfma_v1",
    "mi355_w8a8_calibrate_read_v1", "mi355_w8a8_calibrate_copy_v1",
)

_u32, _u64, _vp, _f32 = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_float


class Problem(ctypes.Structure):
    """struct mi355_w8a8_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("k", _u32), ("n", _u32),
        ("n_adapters", _u32), ("rank", _u32), ("rms_eps", _f32),
        ("x", _vp), ("w_packed", _vp), ("w_scales", _vp), ("lora_a", _vp), ("lora_b", _vp),
        ("lora_scaling", _vp), ("adapter_indices", _vp), ("rms_gamma", _vp), ("residual", _vp),
        ("out", _vp), ("workspace", _vp), ("workspace_bytes", _u64),
        ("aux_x_codes", _vp), ("aux_x_scales", _vp), ("aux_acc", _vp), ("aux_normalized", _vp),
    ]


class GroupedProblem(ctypes.Structure):
    """struct mi355_w8a8_grouped_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("k", _u32), ("n", _u32),
        ("n_groups", _u32), ("rank", _u32), ("groups_per_weight", _u32),
        ("x", _vp), ("w_packed", _vp), ("w_scales", _vp), ("lora_a", _vp), ("lora_b", _vp),
        ("lora_scaling", _vp), ("group_sizes", _vp), ("out", _vp), ("workspace", _vp),
        ("workspace_bytes", _u64), ("aux_x_codes", _vp), ("aux_x_scales", _vp), ("aux_acc", _vp),
        ("x_row_map", _vp), ("x_row_repeat", _u32), ("x_rows", _u32),
    ]


class BwdProblem(ctypes.Structure):
    """struct mi355_w8a8_bwd_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("k", _u32), ("n", _u32),
        ("n_adapters", _u32), ("rank", _u32), ("reserved", _u32),
        ("x", _vp), ("dy", _vp), ("w_packed", _vp), ("w_scales", _vp), ("lora_a", _vp), ("lora_b", _vp),
        ("lora_scaling", _vp), ("adapter_indices", _vp), ("dx", _vp), ("d_lora_a", _vp), ("d_lora_b", _vp),
        ("d_lora_scaling", _vp), ("workspace", _vp), ("workspace_bytes", _u64),
    ]


class GroupedBwdProblem(ctypes.Structure):
    """struct mi355_w8a8_grouped_bwd_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("k", _u32), ("n", _u32),
        ("n_groups", _u32), ("rank", _u32), ("groups_per_weight", _u32),
        ("x", _vp), ("dy", _vp), ("w_packed", _vp), ("w_scales", _vp), ("lora_a", _vp), ("lora_b", _vp),
        ("lora_scaling", _vp), ("group_sizes", _vp), ("dx", _vp), ("d_lora_a", _vp), ("d_lora_b", _vp),
        ("d_lora_scaling", _vp), ("workspace", _vp), ("workspace_bytes", _u64),
    ]


class QkvPostProblem(ctypes.Structure):
    """struct mi355_w8a8_qkv_post_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("num_query_heads", _u32), ("num_kv_heads", _u32),
        ("head_dim", _u32), ("rotary_dim", _u32), ("rope_theta", _f32), ("rms_eps", _f32), ("reserved", _u32),
        ("fused", _vp), ("q_norm_weight", _vp), ("k_norm_weight", _vp), ("positions", _vp),
        ("q", _vp), ("k", _vp), ("v", _vp), ("gate", _vp),
    ]


class QkvPostBwdProblem(ctypes.Structure):
    """struct mi355_w8a8_qkv_post_bwd_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("num_query_heads", _u32), ("num_kv_heads", _u32),
        ("head_dim", _u32), ("rotary_dim", _u32), ("rope_theta", _f32), ("rms_eps", _f32), ("reserved", _u32),
        ("fused", _vp), ("q_norm_weight", _vp), ("k_norm_weight", _vp), ("positions", _vp),
        ("d_q", _vp), ("d_k", _vp), ("d_v", _vp), ("d_gate", _vp), ("d_fused", _vp),
        ("d_q_norm_weight", _vp), ("d_k_norm_weight", _vp), ("workspace", _vp), ("workspace_bytes", _u64),
    ]


class MoeDispatchProblem(ctypes.Structure):
    """struct mi355_w8a8_moe_dispatch_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("n_pairs", _u32), ("repeat", _u32), ("width", _u32),
        ("n_groups", _u32),
        ("tokens", _vp), ("indices", _vp), ("adapter_indices", _vp), ("sorted_tokens", _vp), ("group_sizes", _vp),
        ("sort_indices", _vp), ("unsort_indices", _vp), ("sorted_adapters", _vp), ("workspace", _vp),
        ("workspace_bytes", _u64),
    ]


class GqProblem(ctypes.Structure):
    """struct mi355_w8a8_gq_problem"""

    _fields_ = [
        ("struct_size", _u32), ("flags", _u32), ("m", _u32), ("k", _u32), ("k_pad", _u32), ("n", _u32),
        ("group_size", _u32), ("weight_bits", _u32), ("activation_bits", _u32), ("n_adapters", _u32),
        ("rank", _u32), ("reserved", _u32),
        ("x", _vp), ("w_packed", _vp), ("w_scales", _vp), ("lora_a", _vp), ("lora_b", _vp), ("lora_scaling", _vp),
        ("adapter_indices", _vp), ("out", _vp), ("workspace", _vp), ("workspace_bytes", _u64),
        ("aux_x_codes", _vp), ("aux_x_scales", _vp), ("aux_base", _vp),
    ]


class NativeError(RuntimeError):
    def __init__(self, fn: str, status: int, detail: str):
        super().__init__(f"{fn} failed: {STATUS.get(status, status)} ({detail})")
        self.status = status


_lock = threading.Lock()
_lib = None


def _bind(lib: ctypes.CDLL) -> None:
    lib.mi355_w8a8_abi_version.restype = ctypes.c_int
    lib.mi355_w8a8_abi_version.argtypes = ()
    lib.mi355_w8a8_status_string.restype = ctypes.c_char_p
    lib.mi355_w8a8_status_string.argtypes = (ctypes.c_int,)
    lib.mi355_w8a8_packed_weight_bytes.restype = _u64
    lib.mi355_w8a8_packed_weight_bytes.argtypes = (_u32, _u32)
    for name in ("mi355_w8a8_pack_weight_v1", "mi355_w8a8_unpack_weight_v1"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = (_vp, _vp, _u32, _u32, _vp)
    lib.mi355_w8a8_quantize_rows_v1.restype = ctypes.c_int
    lib.mi355_w8a8_quantize_rows_v1.argtypes = (_vp, _vp, _vp, _u32, _u32, _vp)
    for name in ("mi355_w8a8_workspace_bytes", "mi355_w8a8_grouped_workspace_bytes",
                 "mi355_w8a8_bwd_workspace_bytes"):
        fn = getattr(lib, name)
        fn.restype = _u64
        fn.argtypes = (_u32, _u32, _u32, _u32, _u32, _u32)
    for name in ("mi355_w8a8_lora_linear_v1", "mi355_w8a8_rms_gateup_swiglu_v1",
                 "mi355_w8a8_lora_residual_v1", "mi355_w8a8_forward_v1", "mi355_w8a8_forward_static_ws_v1"):
        fn = getattr(lib, name)
        fn.restype = ctypes.c_int
        fn.argtypes = (ctypes.POINTER(Problem), _vp)
    lib.mi355_w8a8_grouped_v1.restype = ctypes.c_int
    lib.mi355_w8a8_grouped_v1.argtypes = (ctypes.POINTER(GroupedProblem), _vp)
    lib.mi355_w8a8_lora_linear_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_lora_linear_bwd_v1.argtypes = (ctypes.POINTER(BwdProblem), _vp)
    lib.mi355_w8a8_grouped_bwd_workspace_bytes.restype = _u64
    lib.mi355_w8a8_grouped_bwd_workspace_bytes.argtypes = (_u32, _u32, _u32, _u32, _u32, _u32)
    lib.mi355_w8a8_grouped_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_grouped_bwd_v1.argtypes = (ctypes.POINTER(GroupedBwdProblem), _vp)
    lib.mi355_w8a8_qkv_split_norm_rope_v1.restype = ctypes.c_int
    lib.mi355_w8a8_qkv_split_norm_rope_v1.argtypes = (ctypes.POINTER(QkvPostProblem), _vp)
    lib.mi355_w8a8_qkv_bwd_workspace_bytes.restype = _u64
    lib.mi355_w8a8_qkv_bwd_workspace_bytes.argtypes = (_u32, _u32)
    lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_qkv_split_norm_rope_bwd_v1.argtypes = (ctypes.POINTER(QkvPostBwdProblem), _vp)
    lib.mi355_w8a8_delta_rms_norm_bwd_workspace_bytes.restype = _u64
    lib.mi355_w8a8_delta_rms_norm_bwd_workspace_bytes.argtypes = (_u32, _u32)
    lib.mi355_w8a8_delta_rms_norm_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_delta_rms_norm_bwd_v1.argtypes = (_vp, _vp, _vp, _vp, _vp, _vp, _u64, _u32, _u32, _f32, _vp)
    lib.mi355_w8a8_moe_route_v1.restype = ctypes.c_int
    lib.mi355_w8a8_moe_route_v1.argtypes = (_vp, _u32, _u32, _u32, _u32, _vp, _vp, _vp)
    lib.mi355_w8a8_moe_route_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_moe_route_bwd_v1.argtypes = (_vp, _vp, _vp, _u32, _u32, _u32, _u32, _vp, _vp)
    lib.mi355_w8a8_moe_dispatch_workspace_bytes.restype = _u64
    lib.mi355_w8a8_moe_dispatch_workspace_bytes.argtypes = (_u32, _u32)
    lib.mi355_w8a8_moe_dispatch_v1.restype = ctypes.c_int
    lib.mi355_w8a8_moe_dispatch_v1.argtypes = (ctypes.POINTER(MoeDispatchProblem), _vp)
    lib.mi355_w8a8_moe_combine_v1.restype = ctypes.c_int
    lib.mi355_w8a8_moe_combine_v1.argtypes = (_vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp)
    lib.mi355_w8a8_moe_combine_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_moe_combine_bwd_v1.argtypes = (_vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _vp)
    lib.mi355_w8a8_gq_packed_weight_bytes.restype = _u64
    lib.mi355_w8a8_gq_packed_weight_bytes.argtypes = (_u32, _u32, _u32)
    lib.mi355_w8a8_gq_pack_weight_v1.restype = ctypes.c_int
    lib.mi355_w8a8_gq_pack_weight_v1.argtypes = (_vp, _vp, _u32, _u32, _u32, _vp)
    lib.mi355_w8a8_gq_workspace_bytes.restype = _u64
    lib.mi355_w8a8_gq_workspace_bytes.argtypes = (_u32, _u32, _u32, _u32, _u32)
    lib.mi355_w8a8_gq_linear_v1.restype = ctypes.c_int
    lib.mi355_w8a8_gq_linear_v1.argtypes = (ctypes.POINTER(GqProblem), _vp)
    lib.mi355_w8a8_forward_path.restype = ctypes.c_int
    lib.mi355_w8a8_forward_path.argtypes = (_u32, _u32, _u32, _u32)
    lib.mi355_w8a8_calibrate_operand_bytes.restype = _u64
    lib.mi355_w8a8_calibrate_operand_bytes.argtypes = ()
    lib.mi355_w8a8_calibrate_mfma_ops.restype = _u64
    lib.mi355_w8a8_calibrate_mfma_ops.argtypes = (_u32, _u32)
    lib.mi355_w8a8_calibrate_mfma_v1.restype = ctypes.c_int
    lib.mi355_w8a8_calibrate_mfma_v1.argtypes = (_u32, _vp, _u32, _vp, _vp, _vp)
    lib.mi355_w8a8_calibrate_read_v1.restype = ctypes.c_int
    lib.mi355_w8a8_calibrate_read_v1.argtypes = (_vp, _u64, _vp, _vp)
    lib.mi355_w8a8_calibrate_copy_v1.restype = ctypes.c_int
    lib.mi355_w8a8_calibrate_copy_v1.argtypes = (_vp, _vp, _u64, _vp)
    lib.mi355_w8a8_swiglu_v1.restype = ctypes.c_int
    lib.mi355_w8a8_swiglu_v1.argtypes = (_vp, _vp, _u32, _u32, _vp)
    lib.mi355_w8a8_swiglu_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_swiglu_bwd_v1.argtypes = (_vp, _vp, _vp, _u32, _u32, _vp)
    lib.mi355_w8a8_rms_norm_bwd_v1.restype = ctypes.c_int
    lib.mi355_w8a8_rms_norm_bwd_v1.argtypes = (_vp, _vp, _vp, _vp, _u32, _u32, _f32, _vp)


def load() -> ctypes.CDLL:
    """Load (once) and return the native library; raises if it was not built."""
    global _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with skyrl-tx-rocm_amd/build.py "
                    "(there is no CPU fallback for the W8A8 path)")
            lib = ctypes.CDLL(str(LIB_PATH), mode=ctypes.RTLD_LOCAL)
            for name in EXPORTS:
                if not hasattr(lib, name):
                    raise RuntimeError(f"{LIB_PATH} does not export {name}")
            _bind(lib)
            if lib.mi355_w8a8_abi_version() != ABI_VERSION:
                raise RuntimeError("libmi355_w8a8.so ABI version mismatch")
            _lib = lib
        return _lib


def check(fn: str, status: int) -> None:
    if status != 0:
        detail = load().mi355_w8a8_status_string(status).decode()
        raise NativeError(fn, status, detail)
