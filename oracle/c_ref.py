"""ctypes binding of the plain-C restatement (oracle/attn_jvp_ref.c).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import math
import os
import subprocess
from typing import Dict, Optional

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libattn_jvp_ref.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile oracle/attn_jvp_ref.c with gcc (the Makefile beside it)."""
    if force and os.path.exists(_SO):
        os.remove(_SO)
    subprocess.run(["make", "-C", _HERE, "libattn_jvp_ref.so"], check=True, capture_output=True)
    return _SO


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        _lib = ctypes.CDLL(_SO)
        dp = ctypes.POINTER(ctypes.c_double)
        i64 = ctypes.c_int64
        _lib.attn_jvp_ref_forward.argtypes = [dp] * 11 + [i64] * 4 + [ctypes.c_double]
        _lib.attn_jvp_ref_forward.restype = ctypes.c_int
        _lib.attn_jvp_ref_backward.argtypes = [dp] * 18 + [i64] * 4 + [ctypes.c_double]
        _lib.attn_jvp_ref_backward.restype = ctypes.c_int
    return _lib


def _p(a: Optional[np.ndarray]):
    if a is None:
        return None
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_double))


def _c(x) -> np.ndarray:
    import torch
    if isinstance(x, torch.Tensor):
        x = x.detach().to(torch.float64).cpu().numpy()
    return np.ascontiguousarray(x, dtype=np.float64)


def attention_jvp_c(q, k, v, tq, tk, tv, dO=None, dTO=None,
                    scale: Optional[float] = None) -> Dict[str, np.ndarray]:
    """Forward (+ backward when a cotangent is given) through the C restatement; [B,H,L,D] in/out."""
    q, k, v, tq, tk, tv = (_c(x) for x in (q, k, v, tq, tk, tv))
    B, H, Lq, D = q.shape
    Lk = k.shape[2]
    s = 1.0 / math.sqrt(D) if scale is None else float(scale)
    Lr = ((Lq + 127) // 128) * 128
    o = np.empty_like(q)
    to = np.empty_like(q)
    lse = np.empty((B, H, Lr))
    mu = np.empty((B, H, Lr))
    li = np.empty((B, H, Lr))
    L = lib()
    rc = L.attn_jvp_ref_forward(_p(q), _p(k), _p(v), _p(tq), _p(tk), _p(tv), _p(o), _p(to), _p(lse),
                                _p(mu), _p(li), B * H, Lq, Lk, D, s)
    assert rc == 0
    res = {"O": o, "TO": to, "M": lse, "MU": mu, "LI": li}
    if dO is None and dTO is None:
        return res
    dOn = None if dO is None else _c(dO)
    G = None if dTO is None else _c(dTO)
    grads = {n: np.empty_like(q if n in ("dq", "dtq") else k)
             for n in ("dq", "dk", "dv", "dtq", "dtk", "dtv")}
    rc = L.attn_jvp_ref_backward(_p(q), _p(k), _p(v), _p(tq), _p(tk), _p(tv), _p(o), _p(to), _p(dOn),
                                 _p(G), _p(lse), _p(mu), *(_p(grads[n]) for n in
                                                           ("dq", "dk", "dv", "dtq", "dtk", "dtv")),
                                 B * H, Lq, Lk, D, s)
    assert rc == 0
    res.update(grads)
    return res
