"""ctypes binding of libt2fw_hip.so (C ABI declared in include/t2fw_hip.h).

torch is imported first so that the library binds to the HIP runtime torch already
loaded; stream handles from torch are then valid in the library.  There is no CPU
fallback: a missing library is an ImportError-like RuntimeError at first use.
"""
import ctypes
import os

import torch  # noqa: F401  (must be loaded before the HIP library)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libt2fw_hip.so")

ABI_VERSION = 3

F32, F16, BF16, F64 = 0, 1, 2, 3
DTYPE_CODE = {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16, torch.float64: F64}

FLAG_AUTO = 0
FLAG_FORCE_SCAN = 1
FLAG_FP16_OPERANDS = 2
FLAG_NO_FIXUP = 4
FLAG_BLOCKWISE = 8
FLAG_BF16_OPERANDS = 16

_vp, _i64, _i32, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/t2fw_hip.h one to one
SIGNATURES = {
    "t2fw_abi_version": (ctypes.c_int, []),
    "t2fw_last_error": (ctypes.c_char_p, []),
    "t2fw_lfw_num_ckpt": (_i64, [_i64, _i32]),
    "t2fw_lfw_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i32, _i32, _i32]),
    "t2fw_lfw_forward_workspace_bytes": (_sz, [_i64, _i64, _i64, _i64, _i32, _i32, _i32]),
    "t2fw_lfw_flag_regions": (ctypes.c_int, [_i64] * 4 + [_i32] * 3 + [ctypes.POINTER(ctypes.c_int64)]),
    "t2fw_host_workspace_device_pointer": (ctypes.c_int, [_vp, ctypes.POINTER(ctypes.c_void_p)]),
    "t2fw_lfw_forward": (ctypes.c_int, [_vp] * 9 + [_i64] * 4 + [_i32] * 3 + [_vp, _sz, _vp]),
    "t2fw_static_init": (ctypes.c_int, []),
    "t2fw_lfw_forward_static": (ctypes.c_int, [_vp] * 9 + [_i64] * 4 + [_i32] * 3 + [_vp]),
    "t2fw_lfw_backward": (ctypes.c_int, [_vp] * 15 + [_i64] * 4 + [_i32] * 3 + [_vp, _sz, _vp]),
    "t2fw_lfw_forward_heads": (ctypes.c_int, [_vp] * 9 + [_i64] * 5 + [_i32] * 3 + [_vp, _sz, _vp]),
    "t2fw_lfw_backward_heads": (ctypes.c_int, [_vp] * 15 + [_i64] * 5 + [_i32] * 3 + [_vp, _sz, _vp]),
    "t2fw_lfw_step": (ctypes.c_int, [_vp] * 8 + [_i64] * 3 + [_i32, _vp]),
    "t2fw_cast": (ctypes.c_int, [ctypes.POINTER(ctypes.c_void_p)] * 2 + [ctypes.POINTER(ctypes.c_int64), _i32, _i32, _i32, _vp]),
    "t2fw_gate_forward": (ctypes.c_int, [_vp] * 4 + [_i64] * 2 + [_i32, _vp]),
    "t2fw_gate_backward": (ctypes.c_int, [_vp] * 6 + [_i64] * 2 + [_i32, _vp]),
    "t2fw_dfw_forward": (ctypes.c_int, [_vp] * 7 + [_i64] * 4 + [_i32, _i32, _vp]),
    "t2fw_dfw_backward": (ctypes.c_int, [_vp] * 10 + [_i64] * 4 + [_i32, _i32, _vp]),
}

_lib = None


def load():
    """Load the shared library (once).  Raises RuntimeError when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "t2fw: %s is missing -- build it with `python -m t2fw_amd.build` "
            "(there is no CPU fallback)" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    got = lib.t2fw_abi_version()
    if got != ABI_VERSION:
        raise RuntimeError("t2fw: library ABI version %d, binding expects %d" % (got, ABI_VERSION))
    _lib = lib
    return lib


def check(rc):
    """Turn a nonzero return code into RuntimeError carrying the library's message."""
    if rc != 0:
        msg = load().t2fw_last_error()
        raise RuntimeError("t2fw error %d: %s" % (rc, msg.decode() if msg else "?"))


def ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def current_stream_handle(device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def cast_tensors(srcs, dsts, stream):
    """One launch of t2fw_cast: srcs[i] -> dsts[i] elementwise (float32 <-> float16 / bfloat16; every source of
    one dtype, every destination of one dtype; contiguous tensors of equal element counts, at most eight)."""
    lib = load()
    n = len(srcs)
    assert n == len(dsts) and 0 < n <= 8
    for a, b in zip(srcs, dsts):
        assert a.numel() == b.numel() and a.is_contiguous() and b.is_contiguous()
        assert a.dtype == srcs[0].dtype and b.dtype == dsts[0].dtype
    sp = (ctypes.c_void_p * n)(*[ptr(t) for t in srcs])
    dp = (ctypes.c_void_p * n)(*[ptr(t) for t in dsts])
    cnt = (ctypes.c_int64 * n)(*[t.numel() for t in srcs])
    check(lib.t2fw_cast(sp, dp, cnt, n, DTYPE_CODE[srcs[0].dtype], DTYPE_CODE[dsts[0].dtype], stream))
