"""ctypes binding of libsjvp.so (C ABI in include/sjvp.h).  There is no fallback: if the library is
missing or a call fails, an exception is raised."""
from __future__ import annotations

import ctypes
import threading

from . import build as _build

SJVP_BF16 = 0
SJVP_FP16 = 1
SJVP_FP32 = 2
SJVP_FP32_BF16 = 3  # fp32 tensors, bf16 arithmetic (casts folded into loads and stores)

SJVP_OK = 0
SJVP_ERR_NULL = -1
SJVP_ERR_SHAPE = -2
SJVP_ERR_HEAD_DIM = -3
SJVP_ERR_DTYPE = -4
SJVP_ERR_WORKSPACE = -5
SJVP_ERR_LAUNCH = -6
SJVP_ERR_COTANGENT = -7
SJVP_ERR_PARTS = -8
SJVP_ERR_ROTARY = -9
SJVP_ERR_SCALE = -10
SJVP_ERR_SCRATCH = -11
SJVP_NOALLOC_MAX_ROWS = 1 << 20

SJVP_BWD_ROW = 1
SJVP_BWD_COL = 2
SJVP_BWD_ALL = 3

F_TENSORS = ("q", "k", "v", "tq", "tk", "tv", "o", "to")
B_TENSORS = ("q", "k", "v", "tq", "tk", "tv", "o", "to", "dO", "dTO",
             "dq", "dk", "dv", "dtq", "dtk", "dtv")

SJVP_REPAIR_OFF = 0
SJVP_REPAIR_AUTO = 1
SJVP_REPAIR_ALWAYS = 2

EXPORTS = ("sjvp_fwd", "sjvp_bwd", "sjvp_bwd_parts", "sjvp_bwd_noalloc", "sjvp_fwd_rotary", "sjvp_bwd_rotary", "sjvp_bwd_workspace_bytes", "sjvp_rope",
           "sjvp_set_row_sum_repair", "sjvp_strerror", "sjvp_version", "sjvp_build_id")

_lock = threading.Lock()
_lib = None


class SjvpError(RuntimeError):
    def __init__(self, status: int, message: str):
        super().__init__(f"sjvp status {status}: {message}")
        self.status = status


def load() -> ctypes.CDLL:
    """Load the in-tree shared library; it is built first when it does not exist or is older than one
    of its sources (a stale binary is never loaded silently)."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            path = _build.LIB_PATH
            if _build.is_stale():
                _build.build()
            lib = ctypes.CDLL(path)
            vp, fp, i, i64p = ctypes.c_void_p, ctypes.POINTER(ctypes.c_float), ctypes.c_int, \
                ctypes.POINTER(ctypes.c_int64)
            lib.sjvp_fwd.argtypes = [vp] * 8 + [vp] * 3 + [i] * 5 + [i64p, ctypes.c_float, i, vp]
            lib.sjvp_fwd.restype = i
            lib.sjvp_bwd.argtypes = ([vp] * 10 + [vp] * 2 + [vp] * 6 + [vp, ctypes.c_size_t] + [i] * 5 +
                                     [i64p, ctypes.c_float, i, vp])
            lib.sjvp_bwd.restype = i
            lib.sjvp_bwd_noalloc.argtypes = ([vp] * 10 + [vp] * 2 + [vp] * 6 + [i] * 5 +
                                             [i64p, ctypes.c_float, i, vp])
            lib.sjvp_bwd_noalloc.restype = i
            rot = [vp, vp, ctypes.c_int64, i]  # cos, sin, row stride, rows
            lib.sjvp_fwd_rotary.argtypes = ([vp] * 8 + [vp] * 3 + [i] * 5 + [i64p, ctypes.c_float, i] + rot + [vp])
            lib.sjvp_fwd_rotary.restype = i
            lib.sjvp_bwd_rotary.argtypes = ([vp] * 10 + [vp] * 2 + [vp] * 6 + [i] * 5 + [i64p, ctypes.c_float, i] +
                                            rot + [vp])
            lib.sjvp_bwd_rotary.restype = i
            lib.sjvp_bwd_parts.argtypes = [i] + lib.sjvp_bwd.argtypes
            lib.sjvp_bwd_parts.restype = i
            lib.sjvp_bwd_workspace_bytes.argtypes = [i] * 6
            lib.sjvp_bwd_workspace_bytes.restype = ctypes.c_size_t
            vpp = ctypes.POINTER(ctypes.c_void_p)
            lib.sjvp_rope.argtypes = [i, vpp, vpp, i64p, vp, vp, ctypes.c_int64] + [i] * 8 + [vp]
            lib.sjvp_rope.restype = i
            lib.sjvp_set_row_sum_repair.argtypes = [i]
            lib.sjvp_set_row_sum_repair.restype = i
            lib.sjvp_strerror.argtypes = [i]
            lib.sjvp_strerror.restype = ctypes.c_char_p
            lib.sjvp_version.argtypes = []
            lib.sjvp_version.restype = i
            lib.sjvp_build_id.argtypes = []
            lib.sjvp_build_id.restype = ctypes.c_char_p
            if lib.sjvp_build_id().decode() != "SJVP_BUILD_ID=" + _build.source_id():
                raise RuntimeError(f"{path} was built from other sources than the ones in this tree")
            _lib = lib
    return _lib


def strerror(status: int) -> str:
    return load().sjvp_strerror(status).decode()


def check(status: int) -> None:
    if status != SJVP_OK:
        raise SjvpError(status, strerror(status))
