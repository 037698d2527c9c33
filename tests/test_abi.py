"""CPU-side checks of the C-ABI shared library: it loads without a GPU, exports every
symbol include/t2fw_hip.h declares, and rejects bad arguments before touching a
device (no compute calls here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "t2fw_hip.h")


@pytest.fixture(scope="module")
def lib():
    from t2fw_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from t2fw_amd import build
        build.build()
    return _lib.load()


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(t2fw_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for n in ("t2fw_lfw_forward", "t2fw_lfw_backward", "t2fw_lfw_step", "t2fw_dfw_forward",
              "t2fw_dfw_backward", "t2fw_cast", "t2fw_last_error", "t2fw_abi_version", "t2fw_lfw_num_ckpt",
              "t2fw_lfw_workspace_bytes"):
        assert n in names


def test_library_exports_every_declared_symbol(lib):
    for n in declared_functions():
        assert hasattr(lib, n), "symbol %s is declared in the header but not exported" % n


def test_binding_covers_every_declared_symbol():
    from t2fw_amd import _lib
    assert sorted(_lib.SIGNATURES) == declared_functions()


def test_abi_version_and_ckpt_count(lib):
    assert lib.t2fw_abi_version() == 3
    assert lib.t2fw_lfw_num_ckpt(1024, 64) == 16
    assert lib.t2fw_lfw_num_ckpt(1025, 64) == 17
    assert lib.t2fw_lfw_num_ckpt(1, 64) == 1
    assert lib.t2fw_lfw_num_ckpt(0, 64) == 1
    assert lib.t2fw_lfw_num_ckpt(8192, 1) == 8192


def test_workspace_queries(lib):
    fwd = lib.t2fw_lfw_forward_workspace_bytes(96, 1024, 64, 64, 64, 1, 0)
    both = lib.t2fw_lfw_workspace_bytes(96, 1024, 64, 64, 64, 1, 0)
    assert fwd == 2 * 768 and both > 96 * 16 * 8192                      # flags; + per-chunk scratch of the backward
    assert lib.t2fw_lfw_workspace_bytes(96, 1024, 64, 64, 64, 1, 8) == fwd     # block-wise backward: flags only
    assert lib.t2fw_lfw_workspace_bytes(96, 1024, 64, 64, 16, 1, 0) == fwd     # interval the chunk-parallel form does not take
    assert lib.t2fw_lfw_workspace_bytes(96, 1024, 33, 17, 64, 1, 0) == 0       # exact kernels: none
    assert lib.t2fw_lfw_workspace_bytes(96, 1024, 64, 64, 64, 0, 0) == 0       # fp32: exact kernels
    # arrays of 2^31 elements and more are beyond the chunk-parallel kernels' 32-bit offsets: block-wise, flags only
    big = lib.t2fw_lfw_workspace_bytes(4096, 16384, 64, 64, 64, 1, 0)
    assert big == lib.t2fw_lfw_forward_workspace_bytes(4096, 16384, 64, 64, 64, 1, 0)


def _fwd(lib, ptrs, B, T, D, K, C, dtype):
    return lib.t2fw_lfw_forward(*ptrs, B, T, D, K, C, dtype, 0, None, 0, None)


def test_forward_rejects_bad_arguments(lib):
    buf = ctypes.create_string_buffer(4096)
    base = ctypes.addressof(buf)
    base += (-base) % 64
    p = [ctypes.c_void_p(base)] * 9
    assert _fwd(lib, p, 1, 1, 1, 1, 1, 99) == 2                    # bad dtype
    assert b"dtype" in lib.t2fw_last_error()
    assert _fwd(lib, p, -1, 1, 1, 1, 1, 0) == 3                    # bad shape
    assert _fwd(lib, p, 1, 1, 0, 1, 1, 0) == 3
    assert _fwd(lib, p, 1, 1, 1, 1, 0, 0) == 3                     # C < 1 with checkpoints
    assert _fwd(lib, p, 1 << 40, 1 << 20, 1 << 10, 1 << 10, 1, 0) == 3   # not addressable
    nul = list(p)
    nul[5] = None                                                  # s0
    assert _fwd(lib, nul, 1, 1, 1, 1, 1, 0) == 1
    assert b"s0" in lib.t2fw_last_error()
    nul = list(p)
    nul[0] = None                                                  # x
    assert _fwd(lib, nul, 1, 1, 1, 1, 1, 0) == 1
    mis = list(p)
    mis[5] = ctypes.c_void_p(base + 1)
    assert _fwd(lib, mis, 1, 1, 1, 1, 1, 0) == 4                   # misaligned
    assert _fwd(lib, p, 0, 5, 4, 4, 1, 0) == 0                     # B = 0: nothing to do


def test_backward_rejects_bad_arguments(lib):
    buf = ctypes.create_string_buffer(4096)
    base = ctypes.addressof(buf)
    base += (-base) % 64
    p = [ctypes.c_void_p(base)] * 15
    call = lambda ptrs, *a: lib.t2fw_lfw_backward(*ptrs, *a, 0, None, 0, None)
    assert call(p, 1, 1, 1, 1, 1, 7) == 2
    assert call(p, 1, 1, 1, 1, 0, 0) == 3
    nul = list(p)
    nul[9] = None                                                  # d_x
    assert call(nul, 1, 1, 1, 1, 1, 0) == 1
    assert b"d_x" in lib.t2fw_last_error()


def test_wrapper_has_no_cpu_fallback():
    """CPU tensors are refused (the reference's CHECK_CUDA, t2fw/csrc/lfw.cpp:24)."""
    import torch
    from t2fw.functional_lfw import LFWFunction
    x = torch.randn(1, 2, 3)
    k = torch.randn(1, 2, 2)
    with pytest.raises(RuntimeError, match="CUDA"):
        LFWFunction.apply(x, x, k, k, k, torch.randn(1, 3, 2))


def test_missing_library_fails_loudly(monkeypatch):
    from t2fw_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libt2fw_hip.so")
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.load()
