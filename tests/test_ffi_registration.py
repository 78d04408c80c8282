"""The jax.ffi registration path, exercised with a fake JAX and a fake library (no jaxlib,
no GPU), after the pattern of the reference's tests/tx/kernels/rocm/test_gdn_ffi_smoke.py:42-104."""

import types

import pytest

from __graft_entry__ import load_package


class _FakeHandler:
    restype = None
    argtypes = None


class _FakeLibrary:
    def __init__(self, names):
        for n in names:
            setattr(self, n, _FakeHandler())


class _FakeFfi:
    def __init__(self):
        self.registered = []

    def pycapsule(self, handler):
        return ("capsule", handler)

    def register_ffi_target(self, name, capsule, *, platform, api_version):
        self.registered.append((name, capsule[0], platform, api_version))

    def ffi_call(self, *a, **k):  # pragma: no cover - not reached in these tests
        raise AssertionError("no call expected")


@pytest.fixture()
def ffi_mod(monkeypatch, tmp_path):
    load_package()
    from skyrl_tx_rocm_amd.kernels.rocm import w8a8_ffi

    monkeypatch.setattr(w8a8_ffi, "_registered", False)
    monkeypatch.setattr(w8a8_ffi, "_lifetime_handles", [])
    return w8a8_ffi


def test_register_binds_every_target_for_rocm(ffi_mod, monkeypatch, tmp_path):
    fake_lib_file = tmp_path / "libmi355_w8a8_ffi.so"
    fake_lib_file.write_bytes(b"")
    monkeypatch.setattr(ffi_mod, "FFI_LIB_PATH", fake_lib_file)
    lib = _FakeLibrary(ffi_mod.TARGETS)
    monkeypatch.setattr(ffi_mod, "_load_cdll", lambda path: lib)
    monkeypatch.setattr(ffi_mod.ctypes, "CDLL", lambda *a, **k: object())
    jax = types.SimpleNamespace(ffi=_FakeFfi())
    assert ffi_mod.register(jax) == ffi_mod.TARGETS
    assert [r[0] for r in jax.ffi.registered] == list(ffi_mod.TARGETS)
    assert all(r[2] == "ROCM" and r[3] == 1 for r in jax.ffi.registered)
    for name in ffi_mod.TARGETS:
        h = getattr(lib, name)
        assert h.restype is ffi_mod.ctypes.c_void_p and h.argtypes == (ffi_mod.ctypes.c_void_p,)
    assert lib in ffi_mod._lifetime_handles            # the library is never unloaded
    ffi_mod.register(jax)                               # idempotent: no second registration
    assert len(jax.ffi.registered) == len(ffi_mod.TARGETS)


def test_register_fails_loudly(ffi_mod, monkeypatch, tmp_path):
    with pytest.raises(RuntimeError, match="typed-FFI"):
        ffi_mod.register(types.SimpleNamespace())
    monkeypatch.setattr(ffi_mod, "FFI_LIB_PATH", tmp_path / "absent.so")
    with pytest.raises(RuntimeError, match="is missing"):
        ffi_mod.register(types.SimpleNamespace(ffi=_FakeFfi()))
    present = tmp_path / "present.so"
    present.write_bytes(b"")
    monkeypatch.setattr(ffi_mod, "FFI_LIB_PATH", present)
    monkeypatch.setattr(ffi_mod.ctypes, "CDLL", lambda *a, **k: object())
    monkeypatch.setattr(ffi_mod, "_load_cdll", lambda path: _FakeLibrary(ffi_mod.TARGETS[:1]))
    with pytest.raises(RuntimeError, match="handler symbol"):
        ffi_mod.register(types.SimpleNamespace(ffi=_FakeFfi()))


def test_shim_source_obeys_the_handler_rules():
    """Static rules the reference enforces on its FFI sources
    (tests/tx/kernels/rocm/test_gdn_prepare_ffi.py:456-536): no synchronisation, no allocation."""
    from pathlib import Path

    root = Path(__file__).resolve().parents[1] / "skyrl-tx-rocm_amd" / "csrc"
    for src in sorted(root.glob("*")):
        text = src.read_text()
        for banned in ("hipDeviceSynchronize", "hipStreamSynchronize", "hipMalloc", "hipFree", "hipGraph",
                       "-ffast-math"):
            assert banned not in text, (src.name, banned)
    shim = (root / "w8a8_xla_ffi.cc").read_text()
    assert shim.count("XLA_FFI_DEFINE_HANDLER_SYMBOL") == 9
    assert "PlatformStream<hipStream_t>" in shim
