"""CPU-only checks of the C ABI: the library loads, exports every symbol the header
declares, and rejects invalid requests before touching a GPU."""

import ctypes
import re
from pathlib import Path

import pytest

from __graft_entry__ import load_package

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "mi355_w8a8.h"


@pytest.fixture(scope="module")
def native():
    pkg = load_package()
    if not pkg._native.LIB_PATH.exists():
        pytest.skip("libmi355_w8a8.so not built (run __graft_entry__.build())")
    return pkg._native


def _declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(mi355_w8a8_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(native):
    lib = native.load()
    declared = _declared_functions()
    assert len(declared) >= 13
    for name in declared:
        assert hasattr(lib, name), name
    assert sorted(native.EXPORTS) == declared
    assert lib.mi355_w8a8_abi_version() == 1
    assert lib.mi355_w8a8_status_string(0) == b"ok"
    assert b"workspace" in lib.mi355_w8a8_status_string(-5)


def test_struct_sizes_match_header_layout(native):
    # 8 x 4-byte scalars, 11 pointers, u64, 4 pointers
    assert ctypes.sizeof(native.Problem) == 8 * 4 + 11 * 8 + 8 + 4 * 8
    assert ctypes.sizeof(native.GroupedProblem) == 8 * 4 + 9 * 8 + 8 + 3 * 8 + 8 + 2 * 4
    # backward: 8 x 4-byte scalars, 13 pointers, u64
    assert ctypes.sizeof(native.BwdProblem) == 8 * 4 + 13 * 8 + 8


def test_size_queries(native):
    lib = native.load()
    assert lib.mi355_w8a8_packed_weight_bytes(0, 5) == 0
    assert lib.mi355_w8a8_packed_weight_bytes(64, 17) == 128 * 256
    assert lib.mi355_w8a8_packed_weight_bytes(4096, 24576) == 4096 * 24576
    ws = lib.mi355_w8a8_workspace_bytes(4096, 4096, 24576, 8, 32, 0)
    assert ws >= 4096 * 4096 and ws % 256 == 0
    assert lib.mi355_w8a8_workspace_bytes(16, 12288, 4096, 16, 32, 0) > 0
    assert lib.mi355_w8a8_workspace_bytes(0, 64, 64, 0, 0, 0) == 0          # no rows
    assert lib.mi355_w8a8_workspace_bytes(8, 60, 64, 0, 0, 0) == 0          # K not a multiple of 8
    assert lib.mi355_w8a8_workspace_bytes(8, 32768, 64, 0, 0, 0) == 0       # K too large
    assert lib.mi355_w8a8_workspace_bytes(8, 64, 64, 65, 8, 0) == 0         # too many adapters
    assert lib.mi355_w8a8_workspace_bytes(8, 64, 64, 2, 65, 0) == 0         # rank too large


def _problem(native, **kw):
    p = native.Problem()
    p.struct_size = ctypes.sizeof(native.Problem)
    p.m, p.k, p.n = 8, 64, 32
    fake = 0x10000  # never dereferenced: validation fails first
    p.x, p.w_packed, p.w_scales, p.out, p.workspace = fake, fake + 0x100000, fake + 0x200000, fake + 0x300000, fake + 0x400000
    p.workspace_bytes = 1 << 30
    for k, v in kw.items():
        setattr(p, k, v)
    return p


def test_validation_errors_without_a_gpu(native):
    lib = native.load()
    call = lambda p, fn=lib.mi355_w8a8_forward_v1: fn(ctypes.byref(p), None)
    assert lib.mi355_w8a8_forward_v1(None, None) == -1
    assert call(_problem(native, struct_size=12)) == -8
    assert call(_problem(native, m=0)) == -2
    assert call(_problem(native, k=60)) == -7
    assert call(_problem(native, x=None)) == -1
    assert call(_problem(native, out=None)) == -1
    assert call(_problem(native, x=0x10008)) == -3                       # misaligned
    assert call(_problem(native, out=0x10000)) == -4                     # output aliases x
    assert call(_problem(native, workspace=None)) == -5
    assert call(_problem(native, workspace_bytes=16)) == -5
    assert call(_problem(native, n_adapters=1, rank=8)) == -1            # LoRA pointers missing
    assert call(_problem(native, adapter_indices=0x500000)) == -2        # indices without LoRA
    assert call(_problem(native, flags=native.FLAG_SWIGLU, n=31)) == -2
    assert call(_problem(native, flags=native.FLAG_FORCE_TILED | native.FLAG_FORCE_SKINNY)) == -2
    # 33..64 rows over a long K on a cache-resident weight run as 32-row chunks, which keep no stage to rerun
    assert call(_problem(native, m=64, k=4096, flags=native.FLAG_SKIP_PROLOGUE)) == -7
    assert call(_problem(native, m=40, k=4096, flags=native.FLAG_SKIP_GEMM)) == -7
    # entry points insist on their own stage combination
    assert call(_problem(native), lib.mi355_w8a8_rms_gateup_swiglu_v1) == -2
    assert call(_problem(native), lib.mi355_w8a8_lora_residual_v1) == -2
    assert call(_problem(native, rms_gamma=0x600000), lib.mi355_w8a8_lora_linear_v1) == -2
    assert lib.mi355_w8a8_quantize_rows_v1(None, None, None, 4, 64, None) == -1
    assert lib.mi355_w8a8_quantize_rows_v1(0x10000, 0x20000, 0x30000, 4, 60, None) == -7
    assert lib.mi355_w8a8_pack_weight_v1(None, 0x10000, 64, 32, None) == -1
    assert lib.mi355_w8a8_pack_weight_v1(0x10000, 0x10010, 64, 32, None) == -4


def test_backward_validation_errors_without_a_gpu(native):
    lib = native.load()

    def problem(**kw):
        p = native.BwdProblem()
        p.struct_size = ctypes.sizeof(native.BwdProblem)
        p.m, p.k, p.n = 8, 64, 32
        fake = 0x10000  # never dereferenced: validation fails first
        p.dy, p.w_packed, p.w_scales, p.dx, p.workspace = fake, fake + 0x100000, fake + 0x200000, fake + 0x300000, fake + 0x400000
        p.workspace_bytes = 1 << 30
        for k, v in kw.items():
            setattr(p, k, v)
        return p

    call = lambda p: lib.mi355_w8a8_lora_linear_bwd_v1(ctypes.byref(p), None)
    assert lib.mi355_w8a8_lora_linear_bwd_v1(None, None) == -1
    assert call(problem(struct_size=8)) == -8
    assert call(problem(m=0)) == -2
    assert call(problem(n=36)) == -7                                   # N not a multiple of 8
    assert call(problem(k=60)) == -7
    assert call(problem(flags=1)) == -2                                # SwiGLU has no native backward
    assert call(problem(dy=None)) == -1
    assert call(problem(dx=None)) == -1
    assert call(problem(dx=0x10008)) == -3
    assert call(problem(dx=0x10000)) == -4                             # dx aliases dy
    assert call(problem(workspace=None)) == -5
    assert call(problem(workspace_bytes=64)) == -5
    assert call(problem(n_adapters=2, rank=8)) == -1                   # LoRA pointers missing
    assert call(problem(d_lora_a=0x700000)) == -2                      # cotangent wanted without LoRA
    assert call(problem(adapter_indices=0x500000)) == -2
    lora = dict(n_adapters=2, rank=8, lora_a=0x800000, lora_b=0x900000, lora_scaling=0xa00000)
    assert call(problem(**lora, d_lora_a=0xb00000)) == -1              # x is needed for a LoRA cotangent
    assert call(problem(**lora, x=0xc00000, d_lora_a=0x800000)) == -4  # dA aliases A
    assert lib.mi355_w8a8_bwd_workspace_bytes(4096, 4096, 24576, 8, 32, 0) % 256 == 0
    assert lib.mi355_w8a8_bwd_workspace_bytes(4096, 4096, 24576, 8, 32, 0) > 2 * 4096 * 24576
    assert lib.mi355_w8a8_bwd_workspace_bytes(8, 64, 32, 0, 0, 0) > 0
    assert lib.mi355_w8a8_bwd_workspace_bytes(8, 64, 36, 0, 0, 0) == 0
    assert lib.mi355_w8a8_bwd_workspace_bytes(8, 64, 32, 65, 8, 0) == 0


def test_python_surface_fails_loudly_on_cpu(native):
    """There is no CPU fallback: CPU tensors are refused, as is a missing opt-in."""
    import torch

    pkg = load_package()
    w8, ql = pkg.w8a8_lora, pkg.quantized_lora
    w = ql.quantize_frozen_weight(torch.randn(64, 16), bits=8, group_size=64)
    assert w.codes.dtype == torch.int8 and w.scales.dtype == torch.bfloat16 and tuple(w.scales.shape) == (1, 16)
    deq = ql.dequantize_frozen_weight(w)
    assert deq.shape == (64, 16)
    x = torch.zeros(2, 64, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="disabled by default"):
        w8.w8a8_frozen_linear(x, w)
    with pytest.raises(RuntimeError, match="GPU"):
        w8.w8a8_frozen_linear(x, w, enabled=True)
    with pytest.raises(TypeError, match="exact bool"):
        w8.w8a8_frozen_linear(x, w, enabled="yes")
    with pytest.raises(RuntimeError, match="interpret"):
        w8.w8a8_frozen_linear(x, w, enabled=True, interpret=True)
    w64 = ql.quantize_frozen_weight(torch.randn(128, 16), bits=8, group_size=64)
    with pytest.raises(ValueError, match="per-channel"):
        w8.prepare_weight(w64)
    # W4 / grouped scales go to the group-scaled kernels, which refuse CPU tensors just the same
    w4 = ql.quantize_frozen_weight(torch.randn(64, 16), bits=4, group_size=64)
    with pytest.raises(RuntimeError, match="GPU"):
        ql.quantized_lora_linear(x, w4, torch.zeros(64, 4, dtype=torch.bfloat16),
                                 torch.zeros(4, 16, dtype=torch.bfloat16), 1.0)
    with pytest.raises(RuntimeError, match="GPU"):
        ql.quantized_frozen_linear(x, ql.quantize_frozen_weight(torch.randn(64, 16), bits=8, group_size=32),
                                   activation_bits=4)
    with pytest.raises(ValueError, match="bits must be 4 or 8"):
        ql.quantized_frozen_linear(x, w4, activation_bits=5)


def test_host_quantizer_matches_oracle():
    import numpy as np
    import torch

    from oracle import w8a8_oracle as o

    pkg = load_package()
    rng = np.random.default_rng(3)
    wd = rng.standard_normal((70, 13)).astype(np.float32)
    for bits, g in ((8, 10), (4, 14), (8, 70)):
        got = pkg.quantized_lora.quantize_frozen_weight(torch.from_numpy(wd), bits=bits, group_size=g,
                                                        scale_dtype=torch.float32)
        want = o.quantize_frozen_weight(wd, bits=bits, group_size=g, scale_dtype="f32")
        np.testing.assert_array_equal(got.codes.numpy(), want.codes)
        np.testing.assert_array_equal(got.scales.numpy(), want.scales)
        np.testing.assert_array_equal(pkg.quantized_lora.dequantize_frozen_weight(got).numpy(),
                                      o.dequantize_frozen_weight(want))


def test_same_named_fused_entry_points_validate_like_the_reference(native):
    """bf16_rms_gate_up_lora_swiglu_contiguous / bf16_lora_residual keep the reference's surface:
    default off, exact bools, tile keywords checked, a bf16 matrix in the place of the quantized
    kernel refused."""
    import torch

    pkg = load_package()
    gate_up = pkg.bf16_rms_gate_up_lora_swiglu_contiguous.bf16_rms_gate_up_lora_swiglu_contiguous
    down = pkg.bf16_lora_residual.bf16_lora_residual
    ql = pkg.quantized_lora
    x = torch.zeros(2, 64, dtype=torch.bfloat16)
    w = ql.quantize_frozen_weight(torch.randn(64, 16), bits=8, group_size=64, scale_dtype=torch.float32)
    a, b, s = torch.zeros(64, 4, dtype=torch.bfloat16), torch.zeros(4, 16, dtype=torch.bfloat16), 1.0
    delta = torch.zeros(64)
    with pytest.raises(RuntimeError, match="disabled by default"):
        gate_up(x, delta, w, a, b, s)
    with pytest.raises(TypeError, match="exact bool"):
        gate_up(x, delta, w, a, b, s, enabled=1)
    with pytest.raises(RuntimeError, match="interpret"):
        gate_up(x, delta, w, a, b, s, enabled=True, interpret=True)
    with pytest.raises(ValueError, match="block_k"):
        gate_up(x, delta, w, a, b, s, enabled=True, block_k=0)
    with pytest.raises(ValueError, match="eps"):
        gate_up(x, delta, w, a, b, s, enabled=True, eps=0.0)
    with pytest.raises(TypeError, match="GroupQuantizedWeight"):
        gate_up(x, delta, torch.zeros(64, 16, dtype=torch.bfloat16), a, b, s, enabled=True)
    with pytest.raises(RuntimeError, match="GPU"):
        gate_up(x, delta, w, a, b, s, enabled=True)                  # CPU tensors: no CPU path
    res = torch.zeros(2, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="disabled by default"):
        down(x, w, a, b, s, res)
    with pytest.raises(TypeError, match="exact bool"):
        down(x, w, a, b, s, res, enabled=True, pallas_input_vjp="no")
    with pytest.raises(ValueError, match="row_superblock"):
        down(x, w, a, b, s, res, enabled=True, row_superblock=-1)
    with pytest.raises(TypeError, match="GroupQuantizedWeight"):
        down(x, torch.zeros(64, 16, dtype=torch.bfloat16), a, b, s, res, enabled=True)
    with pytest.raises(RuntimeError, match="GPU"):
        down(x, w, a, b, s, res, enabled=True)


def test_bounded_frozen_lora_linear_argument_checks():
    """The reference's argument checks (skyrl/tx/kernels/bounded_lora.py:31-108) before anything touches a GPU."""
    import torch

    from __graft_entry__ import load_package

    pkg = load_package()
    bounded = pkg.bounded_lora.bounded_frozen_lora_linear
    ql = pkg.quantized_lora
    x = torch.zeros((2, 5, 16), dtype=torch.bfloat16)
    w = ql.quantize_frozen_weight(torch.ones((16, 7), dtype=torch.float32), bits=8, group_size=16)
    a = torch.zeros((16, 8), dtype=torch.bfloat16)
    b = torch.zeros((8, 7), dtype=torch.bfloat16)
    with pytest.raises(TypeError, match="token_tile_size must be an integer"):
        bounded(x, w, a, b, 1.0, token_tile_size=True)
    with pytest.raises(ValueError, match=r"token_tile_size must be in \[1, 2048\]"):
        bounded(x, w, a, b, 1.0, token_tile_size=0)
    with pytest.raises(TypeError, match="GroupQuantizedWeight"):
        bounded(x, torch.zeros((16, 7), dtype=torch.bfloat16), a, b, 1.0)
    with pytest.raises(ValueError, match="rank-two"):
        bounded(x, w, a[None], b, 1.0)
    with pytest.raises(ValueError, match=r"lora_a must have shape \(16, 8\)"):
        bounded(x, w, torch.zeros((16, 4), dtype=torch.bfloat16), b, 1.0)
    with pytest.raises(TypeError, match="floating scalar"):
        bounded(x, w, a, b, torch.ones(2))
    with pytest.raises(ValueError, match="residual shape"):
        bounded(x, w, a, b, 1.0, residual=torch.zeros((2, 5, 8), dtype=torch.bfloat16))
    with pytest.raises(TypeError, match="residual dtype"):
        bounded(x, w, a, b, 1.0, residual=torch.zeros((2, 5, 7), dtype=torch.float32))
    with pytest.raises(TypeError, match="x dtype must be BF16"):
        bounded(x.float(), w, a, b, 1.0)

