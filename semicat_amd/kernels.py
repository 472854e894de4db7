"""Kernel-level entry points: torch tensors in, HIP kernels (libsjvp.so, C ABI) launched on the
current stream, nothing synchronised.  These replace the three launch wrappers of
olsdavis/semicat's ``semicat/jvp_utils``:

* :func:`flash_attention_jvp_multihead_kernel_wrapper`  <- ``ryu_triton.py:295-422``
* :func:`flash_jvp_backward`                             <- ``flash_jvp_backward.py:2293-2714``
* :func:`flash_attn_backward`                            <- ``flash_attn_triton.py:974-1093``

plus the fused forms the autograd layer and the benchmark use (:func:`attention_jvp_forward`,
:func:`attention_forward`, :func:`attention_jvp_backward`).  There is no CPU or eager fallback:
tensors that are not on a GPU, or a missing shared library, raise.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Sequence, Tuple

import torch

from . import _lib

# bf16 / fp16: the MFMA kernels (fp32 accumulation).  float32: the fp32 correctness mode of the library
# (fp32 tensors and arithmetic throughout, vector ALUs; about 1e-6 against fp64).
_DTYPES = {torch.bfloat16: _lib.SJVP_BF16, torch.float16: _lib.SJVP_FP16, torch.float32: _lib.SJVP_FP32}


def _scale_arg(scale: Optional[float]) -> float:
    """The C ABI's spelling of the softmax scale: 0.0 selects 1/sqrt(D), which is what ``None`` means
    in the reference wrappers (ryu_triton.py:324-325); anything else must be a positive finite number."""
    if scale is None:
        return 0.0
    scale = float(scale)
    if not (scale > 0.0) or math.isinf(scale):
        raise ValueError(f"scale must be a positive finite number or None, got {scale}")
    return scale


def _rope_args(rope, Lq: int, Lk: int, device):
    """(cos ptr, sin ptr, row stride, rows) of the fp32 ``[rows, 32]`` tables of a folded rotation."""
    cos, sin = rope
    if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.shape != sin.shape or cos.ndim != 2 \
            or cos.shape[1] != 32 or cos.stride(1) != 1 or sin.stride(1) != 1 or cos.stride(0) != sin.stride(0) \
            or cos.device != device or sin.device != device or cos.shape[0] < max(Lq, Lk):
        raise AssertionError("folded rotary embedding: cos/sin must be float32 [>= max(Lq, Lk), 32] tensors on "
                             "the inputs' device with unit column stride and equal row strides")
    return _ptr(cos), _ptr(sin), cos.stride(0), cos.shape[0]


def rotary_fusable(q: torch.Tensor, k: torch.Tensor, cos: torch.Tensor, others: Sequence[torch.Tensor] = (),
                   sin: Optional[torch.Tensor] = None) -> bool:
    """Whether ``[B,H,L,D]`` views q, k (and ``others``: v, tangents) can take the attention kernels
    with the rotary embedding folded in: head dimension 64 rotated as a whole, at most 128 keys,
    16-bit tensors with 16-byte aligned rows, and fp32 tables ``[>= max(Lq, Lk), 32]`` on the same
    device, 16-byte aligned, with unit column stride and equal row strides that are multiples of 4:
    everything ``_rope_args`` and the C ABI (``check_rotary``) would otherwise reject, so that a
    caller who asks first never sees their errors and falls back to ``sjvp_rope`` + the plain op."""
    if not q.is_cuda or q.dtype not in (torch.bfloat16, torch.float16) or q.shape[-1] != 64 or k.shape[-2] > 128:
        return False
    # Alignment is judged from the offset into the storage (allocations start on 256-byte boundaries):
    # under torch.func transforms the tensors are wrappers without an address of their own.
    for table in (cos,) if sin is None else (cos, sin):
        if table.ndim != 2 or table.shape[1] != 32 or table.shape[0] < max(q.shape[-2], k.shape[-2]) \
                or table.dtype != torch.float32 or table.device != q.device or table.stride(0) % 4 \
                or table.stride(0) < 32 or table.stride(1) != 1 or (table.storage_offset() * 4) % 16:
            return False
    if sin is not None and (sin.shape != cos.shape or sin.stride(0) != cos.stride(0)):
        return False
    for t in (q, k, *others):
        if t is None:
            continue
        if t.dtype != q.dtype or t.device != q.device or t.stride(-1) != 1 or (t.storage_offset() * 2) % 16 \
                or any(s % 8 for s in t.stride()[:3]):
            return False
    return True


_REPAIR_MODES = {"off": _lib.SJVP_REPAIR_OFF, "auto": _lib.SJVP_REPAIR_AUTO, "always": _lib.SJVP_REPAIR_ALWAYS}


def set_row_sum_repair(mode: str) -> str:
    """How the backward deals with what the rounding of ``o``, ``to`` leaves in its row sums (the
    reference forms those sums from the probabilities, flash_jvp_backward.py:2012-2290): ``"off"``,
    ``"auto"`` (default: a second launch of the row-owned kernel recomputes dq, dq_dot with the corrected
    sums for the workgroups whose rows need it) or ``"always"`` (for every row, and the row + column
    launches also where the single launch would run).
    Process-wide; returns the previous mode."""
    if mode not in _REPAIR_MODES:
        raise ValueError(f"row-sum repair mode must be one of {sorted(_REPAIR_MODES)}, got {mode!r}")
    prev = _lib.load().sjvp_set_row_sum_repair(_REPAIR_MODES[mode])
    return {v: k for k, v in _REPAIR_MODES.items()}[prev]


def stat_rows(L: int) -> int:
    """Length of the row-statistic buffers: L rounded up to 128 (ryu_triton.py:351)."""
    return ((L + 127) // 128) * 128


class _Launch:
    """A validated call of the C ABI with its arguments already converted: calling it enqueues the
    kernels on the stream that was current when it was planned (a few microseconds of host time,
    for loops that launch the same problem many times).  Keeps the tensors alive."""

    __slots__ = ("_fn", "_args", "_keep")

    def __init__(self, fn, args, keep):
        self._fn, self._args, self._keep = fn, args, keep

    def __call__(self) -> None:
        rc = self._fn(*self._args)
        if rc:
            _lib.check(rc)


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _strides(tensors: Sequence[Optional[torch.Tensor]]):
    flat = []
    for t in tensors:
        flat.extend((0, 0, 0) if t is None else (t.stride(0), t.stride(1), t.stride(2)))
    return (ctypes.c_int64 * len(flat))(*flat)


def _check_bhld(name: str, t: torch.Tensor, shape, dtype, device) -> None:
    if tuple(t.shape) != tuple(shape):
        raise AssertionError(f"{name} shape mismatch: {tuple(t.shape)} != {tuple(shape)}")
    if t.dtype != dtype:
        raise TypeError(f"{name} dtype {t.dtype} != {dtype}")
    if t.device != device:
        raise ValueError(f"{name} is on {t.device}, expected {device}")
    if t.stride(-1) != 1:
        raise AssertionError(f"{name}: the last dimension must have unit stride")


def _require_gpu(q: torch.Tensor, arithmetic: Optional[str] = None) -> int:
    """The C ABI's dtype tag for the tensors of a call.  ``arithmetic="bf16"`` on float32 tensors
    selects SJVP_FP32_BF16: elements are rounded to bf16 as the kernels load them and results are
    stored as float32 (the casts of functional.py:318-322,330-331 folded into the op)."""
    if not q.is_cuda:
        raise RuntimeError("semicat_amd kernels run on an AMD GPU only; got a tensor on "
                           f"{q.device} (there is no CPU fallback)")
    if q.dtype not in _DTYPES:
        raise TypeError(f"attention-JVP kernels support bfloat16, float16 and float32, got {q.dtype}")
    if arithmetic not in (None, "bf16"):
        raise ValueError(f"arithmetic must be None or 'bf16', got {arithmetic!r}")
    if arithmetic == "bf16" and q.dtype == torch.float32:
        return _lib.SJVP_FP32_BF16
    return _DTYPES[q.dtype]


def _stat(buf: Optional[torch.Tensor], name: str, B: int, H: int, Lr: int, device) -> torch.Tensor:
    if buf is None:
        return torch.empty((B, H, Lr), device=device, dtype=torch.float32)
    if tuple(buf.shape) != (B, H, Lr) or buf.dtype != torch.float32 or not buf.is_contiguous():
        raise AssertionError(f"{name} must be a contiguous float32 tensor of shape {(B, H, Lr)}, "
                             f"got {tuple(buf.shape)} {buf.dtype}")
    return buf


def attention_jvp_forward(q, k, v, tq, tk, tv, scale: Optional[float] = None, o=None, to=None,
                          lse=None, mu=None, li=None, with_li: bool = True, arithmetic: Optional[str] = None,
                          rope=None, _plan: bool = False) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor,
                                     Optional[torch.Tensor]]:
    """Fused forward on [B,H,L,D] views: returns (o, to, lse, mu, li); any of them may be passed in
    to be filled in place.  ``with_li=False`` skips the LI statistic (returned as None).
    ``arithmetic="bf16"`` on float32 tensors: see :func:`_require_gpu`.  ``rope=(cos, sin)``: q, k, tq,
    tk are given unrotated and the kernel applies the rotary embedding as it loads them
    (``sjvp_fwd_rotary``; see :func:`rotary_fusable` for the shapes this serves)."""
    dtype_tag = _require_gpu(q, arithmetic)
    B, H, Lq, D = q.shape
    Lk = k.shape[-2]
    if D < 16:
        raise ValueError(f"D_head must be >= 16, got {D}")
    dev, dt = q.device, q.dtype
    _check_bhld("Q", q, (B, H, Lq, D), dt, dev)
    for name, t in (("K", k), ("V", v), ("t_K", tk), ("t_V", tv)):
        _check_bhld(name, t, (B, H, Lk, D), dt, dev)
    _check_bhld("t_Q", tq, (B, H, Lq, D), dt, dev)
    if o is None:
        o = torch.empty((B, H, Lq, D), device=dev, dtype=dt)
    if to is None:
        to = torch.empty((B, H, Lq, D), device=dev, dtype=dt)
    _check_bhld("y", o, (B, H, Lq, D), dt, dev)
    _check_bhld("t_y", to, (B, H, Lq, D), dt, dev)
    Lr = stat_rows(Lq)
    lse = _stat(lse, "M", B, H, Lr, dev)
    mu = _stat(mu, "MU", B, H, Lr, dev)
    li = _stat(li, "LI", B, H, Lr, dev) if (with_li or li is not None) else None
    if B * H * Lq == 0 and not _plan:  # nothing to compute (an empty batch slice): no launch
        return o, to, lse, mu, li
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        args = (_ptr(q), _ptr(k), _ptr(v), _ptr(tq), _ptr(tk), _ptr(tv), _ptr(o), _ptr(to),
                _ptr(lse), _ptr(mu), _ptr(li), B, H, Lq, Lk, D, _strides((q, k, v, tq, tk, tv, o, to)),
                _scale_arg(scale), dtype_tag)
        fn = lib.sjvp_fwd
        if rope is not None:
            args += _rope_args(rope, Lq, Lk, dev)
            fn = lib.sjvp_fwd_rotary
        args += (ctypes.c_void_p(stream),)
        if _plan:
            return _Launch(fn, args, (q, k, v, tq, tk, tv, o, to, lse, mu, li, rope)), (o, to, lse, mu, li)
        rc = fn(*args)
    _lib.check(rc)
    return o, to, lse, mu, li


def attention_forward(q, k, v, scale: Optional[float] = None, o=None, lse=None,
                      arithmetic: Optional[str] = None, rope=None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Primal-only forward (tangent contractions compiled out): returns (o, lse).  ``rope``: as in
    :func:`attention_jvp_forward`."""
    dtype_tag = _require_gpu(q, arithmetic)
    B, H, Lq, D = q.shape
    Lk = k.shape[-2]
    if D < 16:
        raise ValueError(f"D_head must be >= 16, got {D}")
    dev, dt = q.device, q.dtype
    _check_bhld("Q", q, (B, H, Lq, D), dt, dev)
    _check_bhld("K", k, (B, H, Lk, D), dt, dev)
    _check_bhld("V", v, (B, H, Lk, D), dt, dev)
    if o is None:
        o = torch.empty((B, H, Lq, D), device=dev, dtype=dt)
    _check_bhld("y", o, (B, H, Lq, D), dt, dev)
    lse = _stat(lse, "M", B, H, stat_rows(Lq), dev)
    if B * H * Lq == 0:
        return o, lse
    lib = _lib.load()
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        args = (_ptr(q), _ptr(k), _ptr(v), None, None, None, _ptr(o), None, _ptr(lse), None,
                None, B, H, Lq, Lk, D, _strides((q, k, v, None, None, None, o, None)),
                _scale_arg(scale), dtype_tag)
        if rope is not None:
            rc = lib.sjvp_fwd_rotary(*args, *_rope_args(rope, Lq, Lk, dev), ctypes.c_void_p(stream))
        else:
            rc = lib.sjvp_fwd(*args, ctypes.c_void_p(stream))
    _lib.check(rc)
    return o, lse


def attention_jvp_backward(q, k, v, tq, tk, tv, o, to, lse, mu, dO=None, dTO=None,
                           scale: Optional[float] = None, grads=None, workspace=None,
                           parts: int = _lib.SJVP_BWD_ALL, static_scratch: bool = False,
                           arithmetic: Optional[str] = None, rope=None, _plan: bool = False):
    """Backward on [B,H,L,D] views for cotangents ``dO`` (on o) and ``dTO`` (on to); at least one.
    Returns (dq, dk, dv, dtq, dtk, dtv); the last three are None when ``dTO`` is None (then
    tq, tk, tv, to, mu may be None as well).  ``grads`` optionally supplies the six output buffers
    (the tangent three may be None without dTO); ``workspace`` a uint8 device buffer of at least
    ``sjvp_bwd_workspace_bytes`` bytes (allocated here otherwise).  ``parts`` selects the launches
    (profiling only: SJVP_BWD_COL alone needs the workspace an earlier SJVP_BWD_ROW call filled).
    ``static_scratch=True`` takes the ``sjvp_bwd_noalloc`` entry point instead: the workspace is a
    static device array of the library, so with ``grads`` supplied the call allocates nothing; it
    serves up to ``SJVP_NOALLOC_MAX_ROWS`` statistic rows and calls overlapping on one GPU race.
    ``rope=(cos, sin)``: q, k, tq, tk are the unrotated tensors the forward was given with the same
    ``rope``; the gradients returned are those of the unrotated tensors (``sjvp_bwd_rotary``)."""
    dtype_tag = _require_gpu(q, arithmetic)
    if dO is None and dTO is None:
        raise ValueError("attention_jvp_backward needs a cotangent on o, on to, or on both")
    B, H, Lq, D = q.shape
    Lk = k.shape[-2]
    if D > 128:
        raise AssertionError(f"head dimension must be <= 128, got {D}")
    dev, dt = q.device, q.dtype
    has_g = dTO is not None
    _check_bhld("q", q, (B, H, Lq, D), dt, dev)
    _check_bhld("k", k, (B, H, Lk, D), dt, dev)
    _check_bhld("v", v, (B, H, Lk, D), dt, dev)
    _check_bhld("o", o, (B, H, Lq, D), dt, dev)
    if dO is not None:
        if dO.stride(-1) != 1:
            dO = dO.contiguous()
        _check_bhld("do", dO, (B, H, Lq, D), dt, dev)
    if has_g:
        if dTO.stride(-1) != 1:
            dTO = dTO.contiguous()  # flash_jvp_backward.py:2314-2315
        _check_bhld("dto", dTO, (B, H, Lq, D), dt, dev)
        _check_bhld("tq", tq, (B, H, Lq, D), dt, dev)
        _check_bhld("tk", tk, (B, H, Lk, D), dt, dev)
        _check_bhld("tv", tv, (B, H, Lk, D), dt, dev)
        _check_bhld("to", to, (B, H, Lq, D), dt, dev)
    else:
        tq = tk = tv = to = mu = None
    Lr = stat_rows(Lq)
    if tuple(lse.shape) != (B, H, Lr):
        raise AssertionError(f"lse shape {tuple(lse.shape)} != {(B, H, Lr)}")
    lse = _stat(lse, "lse", B, H, Lr, dev)
    if has_g:
        if mu.shape[-1] != Lr:  # flash_jvp_backward.py:2325-2339
            mu = torch.cat([mu, mu.new_zeros((B, H, Lr - mu.shape[-1]))], dim=-1)
        mu = _stat(mu.contiguous(), "mu", B, H, Lr, dev)
    if grads is None:
        dq, dk, dv = torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)
        dtq, dtk, dtv = ((torch.empty_like(tq), torch.empty_like(tk), torch.empty_like(tv))
                         if has_g else (None, None, None))
    else:
        dq, dk, dv, dtq, dtk, dtv = grads
    _check_bhld("dq", dq, (B, H, Lq, D), dt, dev)
    _check_bhld("dk", dk, (B, H, Lk, D), dt, dev)
    _check_bhld("dv", dv, (B, H, Lk, D), dt, dev)
    if has_g:
        _check_bhld("dtq", dtq, (B, H, Lq, D), dt, dev)
        _check_bhld("dtk", dtk, (B, H, Lk, D), dt, dev)
        _check_bhld("dtv", dtv, (B, H, Lk, D), dt, dev)
    else:
        dtq = dtk = dtv = None
    if B * H * Lq == 0 and not _plan:
        return dq, dk, dv, dtq, dtk, dtv
    lib = _lib.load()
    tensors = (q, k, v, tq, tk, tv, o, to, dO, dTO, dq, dk, dv, dtq, dtk, dtv)
    if rope is not None:
        if workspace is not None or parts != _lib.SJVP_BWD_ALL or _plan or static_scratch:
            raise ValueError("rope excludes workspace, parts, static_scratch and planned launches")
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream().cuda_stream
            rc = lib.sjvp_bwd_rotary(*(_ptr(t) for t in tensors[:10]), _ptr(lse), _ptr(mu),
                                     *(_ptr(t) for t in tensors[10:]), B, H, Lq, Lk, D, _strides(tensors),
                                     _scale_arg(scale), dtype_tag, *_rope_args(rope, Lq, Lk, dev),
                                     ctypes.c_void_p(stream))
        _lib.check(rc)
        return dq, dk, dv, dtq, dtk, dtv
    if static_scratch:
        if workspace is not None or parts != _lib.SJVP_BWD_ALL or _plan:
            raise ValueError("static_scratch excludes workspace, parts and planned launches")
        with torch.cuda.device(dev):
            stream = torch.cuda.current_stream().cuda_stream
            rc = lib.sjvp_bwd_noalloc(*(_ptr(t) for t in tensors[:10]), _ptr(lse), _ptr(mu),
                                      *(_ptr(t) for t in tensors[10:]), B, H, Lq, Lk, D, _strides(tensors),
                                      _scale_arg(scale), dtype_tag, ctypes.c_void_p(stream))
        _lib.check(rc)
        return dq, dk, dv, dtq, dtk, dtv
    nbytes = lib.sjvp_bwd_workspace_bytes(B, H, Lq, Lk, D, dtype_tag)
    if workspace is None:
        workspace = torch.empty((nbytes,), device=dev, dtype=torch.uint8)
    elif workspace.dtype != torch.uint8 or workspace.numel() < nbytes or workspace.device != dev:
        raise AssertionError(f"workspace must be a uint8 tensor of >= {nbytes} bytes on {dev}")
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream().cuda_stream
        args = (int(parts), *(_ptr(t) for t in tensors[:10]), _ptr(lse), _ptr(mu),
                *(_ptr(t) for t in tensors[10:]), _ptr(workspace), nbytes, B, H, Lq, Lk, D,
                _strides(tensors), _scale_arg(scale), dtype_tag, ctypes.c_void_p(stream))
        if _plan:
            return (_Launch(lib.sjvp_bwd_parts, args, tensors + (lse, mu, workspace)),
                    (dq, dk, dv, dtq, dtk, dtv))
        rc = lib.sjvp_bwd_parts(*args)
    _lib.check(rc)
    return dq, dk, dv, dtq, dtk, dtv


def plan_forward(*args, **kwargs):
    """attention_jvp_forward with the launch deferred: returns (launch, (o, to, lse, mu, li)), where
    launch() enqueues the forward on the stream current at planning time."""
    return attention_jvp_forward(*args, _plan=True, **kwargs)


def plan_backward(*args, **kwargs):
    """attention_jvp_backward with the launch deferred: returns (launch, (dq, dk, dv, dtq, dtk, dtv))."""
    return attention_jvp_backward(*args, _plan=True, **kwargs)


# ------------------------------------------------------------------------------------------------
# Drop-in replacements with the reference wrappers' own signatures.

def flash_attention_jvp_multihead_kernel_wrapper(Q, K, V, t_Q, t_K, t_V, scale: Optional[float] = None,
                                                 y=None, t_y=None, M=None, MU=None, LI=None,
                                                 return_M: bool = False):
    """Signature of ``flash_attention_jvp_multihead_triton_kernel_wrapper`` (ryu_triton.py:295-309):
    [B,H,L,D] tensors with arbitrary batch/head/sequence strides; returns ``(y, t_y)`` or, with
    ``return_M``, ``(y, t_y, M, MU, LI)``."""
    y, t_y, M, MU, LI = attention_jvp_forward(Q, K, V, t_Q, t_K, t_V, scale=scale, o=y, to=t_y,
                                              lse=M, mu=MU, li=LI)
    return (y, t_y, M, MU, LI) if return_M else (y, t_y)


def _bshd(t: Optional[torch.Tensor]) -> Optional[torch.Tensor]:
    return None if t is None else t.transpose(1, 2)


def flash_jvp_backward(dto, q, k, v, o, tq, tk, tv, lse, mu, li, dq, dk, dv, dtq, dtk, dtv,
                       softmax_scale: Optional[float] = None, *, to=None) -> None:
    """Signature of ``flash_jvp_backward._flash_attn_backward`` (flash_jvp_backward.py:2293-2312):
    every tensor is [B,S,H,D]; fills the six gradients in place for the cotangent ``dto`` on the
    tangent output.  ``li`` is accepted and ignored (it is not needed mathematically).

    The reference never reads its ``o`` argument (its call site passes the tangent output there,
    functional.py:131-149) and recomputes the row sums ``rowsum(dto*O)``, ``rowsum(dto*TO)`` with five
    contractions.  Here they are formed from ``O`` and ``TO`` directly: called with the reference's 17
    positional arguments, ``o`` is ignored as well and both are recomputed with one fused forward
    launch; a caller that still holds them passes the primal output as ``o`` and the tangent output
    as keyword ``to`` and saves that launch."""
    for tan, tan_grad in zip((tq, tk, tv), (dtq, dtk, dtv)):  # flash_jvp_backward.py:2419-2428
        for i in range(tan.dim()):
            if tan.shape[i] != tan_grad.shape[i]:
                raise ValueError(f"Tangent and tangent gradient have different shapes: "
                                 f"{tan.shape} != {tan_grad.shape}")
    scale = softmax_scale or None  # flash_jvp_backward.py:2323: a zero scale means the default
    if to is None:
        o_bh, to_bh, _, _, _ = attention_jvp_forward(_bshd(q), _bshd(k), _bshd(v), _bshd(tq), _bshd(tk),
                                                     _bshd(tv), scale=scale, with_li=False)
    else:
        o_bh, to_bh = _bshd(o), _bshd(to)
    attention_jvp_backward(_bshd(q), _bshd(k), _bshd(v), _bshd(tq), _bshd(tk), _bshd(tv), o_bh,
                           to_bh, lse, mu, dO=None, dTO=_bshd(dto), scale=scale,
                           grads=tuple(_bshd(g) for g in (dq, dk, dv, dtq, dtk, dtv)))


def flash_attn_backward(do, q, k, v, o, lse, dq, dk, dv, bias=None, causal: bool = False,
                        softmax_scale: Optional[float] = None) -> None:
    """Signature of ``flash_attn_triton._flash_attn_backward`` (flash_attn_triton.py:974-976) as
    semicat calls it (functional.py:192-205: no bias, non-causal): [B,S,H,D] tensors, fills
    dq, dk, dv in place for the cotangent ``do`` on the primal output."""
    if bias is not None or causal:
        raise NotImplementedError("the attention-JVP path is non-causal and bias-free")
    attention_jvp_backward(_bshd(q), _bshd(k), _bshd(v), None, None, None, _bshd(o), None, lse, None,
                           dO=_bshd(do), dTO=None, scale=softmax_scale or None,
                           grads=(_bshd(dq), _bshd(dk), _bshd(dv), None, None, None))


_ROPE_DTYPES = {torch.bfloat16: _lib.SJVP_BF16, torch.float16: _lib.SJVP_FP16, torch.float32: _lib.SJVP_FP32}


def rotary_embedding(xs: Sequence[torch.Tensor], cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                     out_dtype: Optional[torch.dtype] = None, inverse: bool = False
                     ) -> Tuple[torch.Tensor, ...]:
    """Rotary position embedding of up to four ``[B,S,H,D]`` tensors of one shape and dtype in one
    launch (``sjvp_rope``), pairing column ``i`` with ``i + rot/2`` as duo.py:45-55 does through
    flash_attn's ``apply_rotary_emb_torch``; ``cos``/``sin`` are fp32 ``[S, rot/2]`` (any row
    stride).  Inputs may be any views with unit last stride; the results are fresh contiguous
    ``[B,S,H,D]`` tensors of ``out_dtype`` (default: the input dtype).  ``inverse`` applies the
    inverse rotation (the transpose of the map, which is what back-propagates a cotangent).
    ``cos = sin = None``: no rotation, only the cast and the change of layout (one launch for up to
    four tensors: the casts of functional.py:318-322,330-331 around the op for float32 callers)."""
    xs = tuple(xs)
    if not 1 <= len(xs) <= 4:
        raise ValueError("rotary_embedding takes one to four tensors")
    x0 = xs[0]
    if not x0.is_cuda:
        raise RuntimeError("semicat_amd kernels run on an AMD GPU only; got a tensor on "
                           f"{x0.device} (there is no CPU fallback)")
    out_dtype = out_dtype or x0.dtype
    if x0.dtype not in _ROPE_DTYPES or out_dtype not in _ROPE_DTYPES:
        raise TypeError(f"rotary_embedding supports bfloat16, float16 and float32, got {x0.dtype} -> {out_dtype}")
    B, S, H, D = x0.shape
    for x in xs:
        if tuple(x.shape) != (B, S, H, D) or x.dtype != x0.dtype or x.device != x0.device:
            raise AssertionError("rotary_embedding: all tensors must share shape, dtype and device")
        if x.stride(-1) != 1:
            raise AssertionError("rotary_embedding: the last dimension must have unit stride")
    if (cos is None) != (sin is None):
        raise AssertionError("cos and sin come together")
    half = 0 if cos is None else cos.shape[-1]
    if cos is not None:
        if cos.shape != sin.shape or cos.ndim != 2 or cos.shape[0] < S or 2 * half > D:
            raise AssertionError(f"cos/sin must be [>= {S}, rot/2] with rot <= {D}, got {tuple(cos.shape)}")
        if cos.dtype != torch.float32 or sin.dtype != torch.float32 or cos.stride(1) != 1 or sin.stride(1) != 1 \
                or cos.stride(0) != sin.stride(0) or cos.device != x0.device or sin.device != x0.device:
            raise AssertionError("cos/sin must be float32 tensors on the inputs' device with unit column "
                                 "stride and equal row strides")
    ys = tuple(torch.empty((B, S, H, D), device=x0.device, dtype=out_dtype) for _ in xs)
    if B * S * H == 0:
        return ys
    n = len(xs)
    flat = []
    for x, y in zip(xs, ys):  # the C ABI speaks [B,H,L,D]: (batch, head, sequence) strides
        flat.extend((x.stride(0), x.stride(2), x.stride(1), y.stride(0), y.stride(2), y.stride(1)))
    xp = (ctypes.c_void_p * n)(*[x.data_ptr() for x in xs])
    yp = (ctypes.c_void_p * n)(*[y.data_ptr() for y in ys])
    lib = _lib.load()
    with torch.cuda.device(x0.device):
        stream = torch.cuda.current_stream().cuda_stream
        rc = lib.sjvp_rope(n, xp, yp, (ctypes.c_int64 * len(flat))(*flat), _ptr(cos), _ptr(sin),
                           0 if cos is None else cos.stride(0), B, H, S, D, 2 * half, _ROPE_DTYPES[x0.dtype],
                           _ROPE_DTYPES[out_dtype], 1 if inverse else 0, ctypes.c_void_p(stream))
    _lib.check(rc)
    return ys

