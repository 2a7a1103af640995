"""ctypes binding of libma_hip.so (the C ABI declared in include/ma_hip.h).

Only plain pointers and integers cross this boundary; PyTorch is used by the
caller for device memory and streams.  The library is looked up in-tree
(``<package root>/lib/libma_hip.so``, or ``$MA_HIP_LIBRARY``); a missing
library is an error, there is no fallback path.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

ABI_VERSION = 2

MA_F32, MA_F16, MA_BF16 = 0, 1, 2
VARIANTS = {"auto": 0, "generic": 1, "staged": 2, "fused": 3, "resident": 4, "chained": 5}
VARIANT_NAMES = {v: k for k, v in VARIANTS.items()}

MA_OK = 0
MA_ERR_NULL, MA_ERR_SHAPE, MA_ERR_DTYPE, MA_ERR_STRIDE = -1, -2, -3, -4
MA_ERR_WORKSPACE, MA_ERR_UNSUPPORTED, MA_ERR_VARIANT, MA_ERR_DEVICE = -5, -6, -7, -8
MA_ERR_STATIC_LIMIT = -9
MA_ERR_BUSY = -10
MA_STATIC_WORKSPACE_BYTES = 32 << 20


class FwdParams(C.Structure):
    """struct ma_fwd_params"""
    _fields_ = [
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("mask", C.c_void_p),
        ("out", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
        ("E", C.c_int32), ("H", C.c_int32), ("N", C.c_int32), ("D", C.c_int32), ("Dv", C.c_int32),
        ("B", C.c_int32), ("T", C.c_int32), ("pre_pad", C.c_int32),
        ("dtype_qk", C.c_int32), ("dtype_v", C.c_int32), ("variant", C.c_int32), ("flags", C.c_int32),
        ("q_stride", C.c_int64 * 3), ("k_stride", C.c_int64 * 3), ("v_stride", C.c_int64 * 3),
        ("out_stride", C.c_int64 * 3), ("mask_stride", C.c_int64 * 2),
        ("eps", C.c_float), ("mask_dtype", C.c_int32), ("error_word", C.c_void_p),
    ]


class BwdParams(C.Structure):
    """struct ma_bwd_params"""
    _fields_ = [
        ("fwd", FwdParams), ("dout", C.c_void_p), ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("dout_stride", C.c_int64 * 3), ("dq_stride", C.c_int64 * 3), ("dk_stride", C.c_int64 * 3),
        ("dv_stride", C.c_int64 * 3),
    ]


class WsLayout(C.Structure):
    """struct ma_ws_layout (byte offsets into the workspace)"""
    _fields_ = [(n, C.c_uint64) for n in ("aR", "cR", "aL", "cL", "Y", "stats", "sync", "total")]


MA_MASK_U8, MA_MASK_I16, MA_MASK_I32, MA_MASK_I64, MA_MASK_F16, MA_MASK_BF16, MA_MASK_F32, MA_MASK_F64 = range(8)
MA_FLAG_SYNC_READY = 1
MA_FLAG_TEST_NO_SPIN = 2
MA_FLAG_DEVICE_EXCLUSIVE = 4

EXPORTS = ("ma_abi_version", "ma_strerror", "ma_fwd_workspace_layout", "ma_fwd_workspace_bytes",
           "ma_workspace_init", "ma_fwd_select_variant", "ma_fwd_kernel_name", "ma_fwd", "ma_fwd_static", "ma_r_step", "ma_l_step", "ma_z_step",
           "ma_matrix", "ma_bwd_workspace_bytes", "ma_bwd")

_lock = threading.Lock()
_lib = None


def library_path() -> str:
    env = os.environ.get("MA_HIP_LIBRARY")
    if env:
        return env
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    return os.path.join(root, "lib", "libma_hip.so")


def load() -> C.CDLL:
    """Load the library once and declare the prototypes."""
    global _lib
    with _lock:
        if _lib is not None:
            return _lib
        path = library_path()
        if not os.path.exists(path):
            raise ImportError(
                f"libma_hip.so not found at {path}: build it with "
                f"`python monarch-attention_amd/build.py` (hipcc, gfx950)")
        lib = C.CDLL(path)
        P = C.POINTER(FwdParams)
        lib.ma_abi_version.restype = C.c_int
        lib.ma_abi_version.argtypes = []
        lib.ma_strerror.restype = C.c_char_p
        lib.ma_strerror.argtypes = [C.c_int]
        lib.ma_fwd_workspace_layout.restype = C.c_int
        lib.ma_fwd_workspace_layout.argtypes = [P, C.POINTER(WsLayout)]
        lib.ma_fwd_workspace_bytes.restype = C.c_uint64
        lib.ma_fwd_workspace_bytes.argtypes = [P]
        lib.ma_workspace_init.restype = C.c_int
        lib.ma_workspace_init.argtypes = [P, C.c_void_p]
        lib.ma_fwd_select_variant.restype = C.c_int
        lib.ma_fwd_select_variant.argtypes = [P]
        lib.ma_fwd_kernel_name.restype = C.c_char_p
        lib.ma_fwd_kernel_name.argtypes = [P]
        lib.ma_fwd.restype = C.c_int
        lib.ma_fwd.argtypes = [P, C.c_void_p]
        lib.ma_fwd_static.restype = C.c_int
        lib.ma_fwd_static.argtypes = [P, C.c_void_p]
        lib.ma_r_step.restype = C.c_int
        lib.ma_r_step.argtypes = [P, C.c_int, C.c_int, C.c_void_p]
        lib.ma_l_step.restype = C.c_int
        lib.ma_l_step.argtypes = [P, C.c_void_p]
        lib.ma_z_step.restype = C.c_int
        lib.ma_z_step.argtypes = [P, C.c_void_p]
        lib.ma_matrix.restype = C.c_int
        lib.ma_matrix.argtypes = [P, C.c_void_p, C.c_void_p]
        lib.ma_bwd_workspace_bytes.restype = C.c_uint64
        lib.ma_bwd_workspace_bytes.argtypes = [C.POINTER(BwdParams)]
        lib.ma_bwd.restype = C.c_int
        lib.ma_bwd.argtypes = [C.POINTER(BwdParams), C.c_void_p]
        got = lib.ma_abi_version()
        if got != ABI_VERSION:
            raise ImportError(f"libma_hip.so has ABI version {got}, this binding needs {ABI_VERSION}")
        _lib = lib
        return lib


def strerror(status: int) -> str:
    return load().ma_strerror(status).decode()


def check(status: int, what: str) -> None:
    """Raise for a non-zero status of the C layer."""
    if status == MA_OK:
        return
    msg = f"{what}: {strerror(status)} (status {status})"
    if status in (MA_ERR_SHAPE, MA_ERR_DTYPE, MA_ERR_STRIDE, MA_ERR_VARIANT, MA_ERR_NULL):
        raise ValueError(msg)
    if status == MA_ERR_UNSUPPORTED:
        raise NotImplementedError(msg)
    raise RuntimeError(msg)
