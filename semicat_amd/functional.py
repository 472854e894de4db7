"""Autograd surface of the attention-JVP op: ``sdpa_jvp`` / ``safe_sdpa_jvp`` with the semantics of
olsdavis/semicat's ``semicat/jvp_utils/functional.py`` (cited by line below), backed by the HIP
kernels in :mod:`semicat_amd.kernels`.

How the op is wired (same shape as the reference, functional.py:216-307):

* ``SDPAFunction.forward`` only allocates the primal output ``y`` and the statistic ``M``
  (functional.py:218-231); under forward-mode AD its ``jvp`` runs the fused kernel once, which
  fills ``y`` and ``M`` in place and returns the tangent ``t_y`` (functional.py:240-258).
* ``SDPAJVPForwardFunction`` is the reverse-mode node of the tangent output: its backward receives
  the cotangent on ``t_y`` and returns gradients for q, k, v and the three tangents
  (functional.py:52-87).
* ``SDPAFunction.backward`` is the reverse-mode node of the primal output (functional.py:261-268).

Beyond the reference: called without forward-mode tangents the reference returns an uninitialised
``y`` (functional.py:286-287); here that case is detected and a primal-only kernel computes ``y``
(and supports reverse mode), so the op is a strict superset.  A missing tangent is treated as zero.

Two wirings of the same op exist; ``AUTOGRAD_WIRING`` selects the one ``sdpa_jvp`` uses:

* ``"fused"`` (default): the dual inputs are unpacked, ONE autograd node (``SDPAFusedFunction``)
  produces ``y`` and ``t_y`` with one forward launch, and the two are handed back as a dual tensor.
  Reverse mode then reaches that node once, with the cotangents of both outputs, and runs the
  backward as ONE launch (the six gradients are accumulated in fp32 and rounded once).
* ``"reference"``: the reference's three-function arrangement as described above, in which the node
  of ``y`` and the node of ``t_y`` each launch the backward with their own cotangent and autograd
  adds the two 16-bit results for q, k, v.
"""
from __future__ import annotations

from typing import Any, Optional

import torch
import torch.autograd.forward_ad as fwAD
from torch import Tensor

from . import kernels


AUTOGRAD_WIRING = "fused"  # or "reference"
# How safe_sdpa_jvp serves float32 callers with bf16 arithmetic (functional.py:318-332):
#   "torch"   (default) torch casts around the 16-bit LDS-DMA kernels, as the reference does;
#   "library" the library's multi-tensor cast launches around them (half the launches, no kernel that is
#             not the library's own; the same speed on large problems, more host time on small ones);
#   "folded"  the float32 tensors handed to the kernels, which round as they load and store float32
#             (SJVP_FP32_BF16: register-staged kernels, no cast at all, but 1.1 to 2.4 times slower).
# Measured on an MI355X, forward + backward in microseconds, 16-bit callers / torch / library / folded:
#   B=64 H=12 L=128 D=64: 70 / 218 / 207 / 244;  B=128 H=12 L=256: 502 / 936 / 934 / 1609;
#   B=8 H=16 L=1024: 514 / 687 / 668 / 1614;  B=2 H=4 L=256 (host-bound): 41 / 76 / 212 / 86.
FP32_CALLERS = "torch"


def _has_tangent(t: Tensor) -> bool:
    return fwAD.unpack_dual(t).tangent is not None


class SDPAJVPFlashBackwardFunction(torch.autograd.Function):
    """Gradients for the cotangent on the tangent output (functional.py:90-168)."""

    @staticmethod
    def forward(ctx, q, k, v, t_q, t_k, t_v, tangents_t_o, lse, mu, o, t_o):
        dq, dk, dv, dtq, dtk, dtv = kernels.attention_jvp_backward(
            q, k, v, t_q, t_k, t_v, o, t_o, lse, mu, dO=None, dTO=tangents_t_o)
        return dq, dk, dv, dtq, dtk, dtv

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("double backward of the attention-JVP op is not implemented")


class SDPABackwardFunction(torch.autograd.Function):
    """Gradients for the cotangent on the primal output (functional.py:171-213)."""

    @staticmethod
    def forward(ctx, q, k, v, o, do, M, arith=None, cos=None, sin=None):
        dq, dk, dv, _, _, _ = kernels.attention_jvp_backward(
            q, k, v, None, None, None, o, None, M, None, dO=do, dTO=None, arithmetic=arith,
            rope=None if cos is None else (cos, sin))
        return dq, dk, dv

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("double backward of the attention-JVP op is not implemented")


class SDPAJVPForwardFunction(torch.autograd.Function):
    """Runs the fused forward; node of the tangent output (functional.py:52-87)."""

    @staticmethod
    def forward(q, k, v, t_q, t_k, t_v, y, M):
        # y and M (allocated by SDPAFunction.forward) are filled in place by the fused kernel.
        # LI, which the reference also keeps (functional.py:57-59), is not needed by the backward.
        with torch.no_grad():
            # the tangent output takes the memory layout of the primal output
            _, t_y, _, MU, _ = kernels.attention_jvp_forward(q, k, v, t_q, t_k, t_v, o=y,
                                                             to=torch.empty_like(y), lse=M, with_li=False)
        return t_y, MU

    @staticmethod
    def setup_context(ctx, inputs: tuple[Any, ...], output: Any) -> Any:
        t_y, MU = output
        ctx.save_for_backward(*inputs, t_y, MU)
        ctx.mark_non_differentiable(MU)

    @staticmethod
    def backward(ctx, d_t_y, *args):
        q, k, v, t_q, t_k, t_v, y, M, t_y, MU = ctx.saved_tensors
        if d_t_y is None:
            return (None,) * 8
        grads = SDPAJVPFlashBackwardFunction.apply(q, k, v, t_q, t_k, t_v, d_t_y, M, MU, y, t_y)
        return *grads, None, None


def _empty_output(q: Tensor, d_v: int, seq_major: bool) -> Tensor:
    """A ``[B,H,S,D]`` output buffer: contiguous as the reference allocates it (functional.py:224-227),
    or, for callers that work in ``[B,S,H,D]``, a view of a ``[B,S,H,D]``-contiguous buffer, so that
    handing the result back in their layout needs no copy (the kernels write through strides)."""
    B, H, S, _ = q.shape
    if seq_major:
        return torch.empty((B, S, H, d_v), device=q.device, dtype=q.dtype).transpose(1, 2)
    return torch.empty((B, H, S, d_v), device=q.device, dtype=q.dtype)


class SDPAFunction(torch.autograd.Function):
    """The op under forward-mode AD (functional.py:216-268)."""

    @staticmethod
    def forward(q, k, v, seq_major=False):
        y = _empty_output(q, v.shape[-1], seq_major)
        M = torch.empty((q.shape[0], q.shape[1], kernels.stat_rows(q.shape[2])), device=q.device,
                        dtype=torch.float32)
        return y, M

    @staticmethod
    def setup_context(ctx: Any, inputs: tuple[Any, ...], output: Any) -> Any:
        ctx.save_for_forward(*inputs[:3], *output)
        ctx.save_for_backward(*inputs[:3], *output)
        ctx.set_materialize_grads(False)

    @staticmethod
    def jvp(ctx, t_q, t_k, t_v, *_):
        q, k, v, y, M = ctx.saved_for_forward
        t_q = torch.zeros_like(q) if t_q is None else t_q
        t_k = torch.zeros_like(k) if t_k is None else t_k
        t_v = torch.zeros_like(v) if t_v is None else t_v
        t_y, _ = SDPAJVPForwardFunction.apply(q, k, v, t_q, t_k, t_v, y, M)
        return t_y, torch.zeros_like(M)

    @staticmethod
    def backward(ctx, d_y, d_M):
        if d_y is None:
            return None, None, None, None
        q, k, v, y, M = ctx.saved_tensors
        with torch.no_grad():
            dq, dk, dv = SDPABackwardFunction.apply(q, k, v, y, d_y, M)
        return dq, dk, dv, None


class SDPAFusedFunction(torch.autograd.Function):
    """``(q, k, v, t_q, t_k, t_v) -> (y, t_y)`` as one autograd node: one fused forward launch, and
    in reverse mode one backward launch that takes the cotangents of both outputs (either may be
    absent).  Replaces the pair functional.py:52-87 / 216-268 when the caller's dual tensors are
    unpacked by hand (see ``_sdpa``)."""

    @staticmethod
    def forward(q, k, v, t_q, t_k, t_v, seq_major=False, arith=None, cos=None, sin=None):
        y = _empty_output(q, v.shape[-1], seq_major)
        y, t_y, M, MU, _ = kernels.attention_jvp_forward(q, k, v, t_q, t_k, t_v, o=y, to=torch.empty_like(y),
                                                         with_li=False, arithmetic=arith,
                                                         rope=None if cos is None else (cos, sin))
        return y, t_y, M, MU

    @staticmethod
    def setup_context(ctx: Any, inputs: tuple[Any, ...], output: Any) -> Any:
        y, t_y, M, MU = output
        ctx.rope = inputs[8] is not None
        ctx.save_for_backward(*inputs[:6], y, t_y, M, MU, *(inputs[8:10] if ctx.rope else ()))
        ctx.arith = inputs[7]
        ctx.mark_non_differentiable(M, MU)
        ctx.set_materialize_grads(False)

    @staticmethod
    def backward(ctx, d_y, d_t_y, *_):
        if d_y is None and d_t_y is None:
            return (None,) * 10
        q, k, v, t_q, t_k, t_v, y, t_y, M, MU, *rope = ctx.saved_tensors
        cos, sin = rope if ctx.rope else (None, None)
        with torch.no_grad():
            if d_t_y is None:
                dq, dk, dv = SDPABackwardFunction.apply(q, k, v, y, d_y, M, ctx.arith, cos, sin)
                return dq, dk, dv, None, None, None, None, None, None, None
            grads = SDPAJVPFusedBackwardFunction.apply(q, k, v, t_q, t_k, t_v, y, t_y, M, MU, d_y, d_t_y,
                                                       ctx.arith, cos, sin)
        return *grads, None, None, None, None


class SDPAJVPFusedBackwardFunction(torch.autograd.Function):
    """Gradients for cotangents on both outputs in one launch (``d_y`` may be None)."""

    @staticmethod
    def forward(ctx, q, k, v, t_q, t_k, t_v, y, t_y, M, MU, d_y, d_t_y, arith=None, cos=None, sin=None):
        return kernels.attention_jvp_backward(q, k, v, t_q, t_k, t_v, y, t_y, M, MU, dO=d_y, dTO=d_t_y,
                                              arithmetic=arith, rope=None if cos is None else (cos, sin))

    @staticmethod
    def backward(ctx, *grads):
        raise NotImplementedError("double backward of the attention-JVP op is not implemented")


class SDPAPrimalFunction(torch.autograd.Function):
    """The op without forward-mode tangents: plain attention with the primal-only kernels."""

    @staticmethod
    def forward(ctx, q, k, v, seq_major=False, arith=None, cos=None, sin=None):
        rope = None if cos is None else (cos, sin)
        y, M = kernels.attention_forward(q, k, v, o=_empty_output(q, v.shape[-1], seq_major), arithmetic=arith,
                                         rope=rope)
        ctx.save_for_backward(q, k, v, y, M, *(rope or ()))
        ctx.arith = arith
        return y

    @staticmethod
    def backward(ctx, d_y):
        q, k, v, y, M, *rope = ctx.saved_tensors
        dq, dk, dv = SDPABackwardFunction.apply(q, k, v, y, d_y, M, ctx.arith, *rope)
        return dq, dk, dv, None, None, None, None


@torch._dynamo.disable
def sdpa_jvp(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """Fused scaled-dot-product attention with forward-mode (jvp) support; ``[B,H,S,D]`` bf16/fp16
    (functional.py:272-307).  Usage: ``y, t_y = torch.func.jvp(sdpa_jvp, (q, k, v), (t_q, t_k, t_v))``
    or wrap a whole model that calls it in ``torch.func.jvp``; both outputs support ``backward``."""
    return _sdpa(q, k, v, seq_major=False)


@torch._dynamo.disable
def _sdpa(q: Tensor, k: Tensor, v: Tensor, seq_major: bool, arith: Optional[str] = None,
          cos: Optional[Tensor] = None, sin: Optional[Tensor] = None) -> Tensor:
    if _has_tangent(q) or _has_tangent(k) or _has_tangent(v):
        if AUTOGRAD_WIRING == "reference":
            if cos is not None:
                raise ValueError("the reference wiring has no folded rotary embedding")
            y, _ = SDPAFunction.apply(q, k, v, seq_major)
            return y
        (q, t_q), (k, t_k), (v, t_v) = (fwAD.unpack_dual(t) for t in (q, k, v))
        t_q = torch.zeros_like(q) if t_q is None else t_q
        t_k = torch.zeros_like(k) if t_k is None else t_k
        t_v = torch.zeros_like(v) if t_v is None else t_v
        y, t_y, _, _ = SDPAFusedFunction.apply(q, k, v, t_q, t_k, t_v, seq_major, arith, cos, sin)
        return fwAD.make_dual(y, t_y)
    return SDPAPrimalFunction.apply(q, k, v, seq_major, arith, cos, sin)


def safe_sdpa_jvp(q: Tensor, k: Tensor, v: Tensor, precise: bool = False) -> Tensor:
    """``[B,S,H,D]`` wrapper with the reference's dtype policy (functional.py:310-332): inputs that
    are neither bf16 nor fp16 are computed in bfloat16 and the result comes back in their dtype, cast
    with torch as in the reference; for float32 inputs ``FP32_CALLERS`` selects two other routes (the
    library's own cast launches, or float32 tensors handed to the kernels as they are), both measured
    slower or equal (figures beside ``FP32_CALLERS``).  ``precise=True`` runs float32 inputs in the
    library's fp32 mode instead (fp32 arithmetic throughout, about 1e-6 against fp64, much slower
    than the MFMA kernels)."""
    orig_dtype = q.dtype
    arith = None
    fp32_bf16 = orig_dtype == torch.float32 and not precise and AUTOGRAD_WIRING != "reference" \
        and k.dtype == torch.float32 and v.dtype == torch.float32
    if fp32_bf16 and FP32_CALLERS == "library" and q.is_cuda:
        from .rotary import cast_tensors
        q, k, v = cast_tensors((q, k, v), torch.bfloat16)
        y = _sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), seq_major=True).transpose(1, 2)
        return cast_tensors(y, orig_dtype)
    if fp32_bf16 and FP32_CALLERS == "folded":
        arith = "bf16"
    elif orig_dtype != torch.bfloat16 and orig_dtype != torch.float16 and not (precise and orig_dtype == torch.float32):
        q = q.to(torch.bfloat16)
        k = k.to(torch.bfloat16)
        v = v.to(torch.bfloat16)
    # The reference returns a [B,S,H,D] view of a [B,H,S,D]-contiguous result, which its callers then
    # copy when they flatten the heads (duo.py:155); here the kernels write [B,S,H,D] memory directly.
    y = _sdpa(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), seq_major=True, arith=arith).transpose(1, 2)
    if y.dtype != orig_dtype:
        y = y.to(orig_dtype)
    return y


@torch._dynamo.disable
def safe_sdpa_jvp_rotary(q: Tensor, k: Tensor, v: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """``safe_sdpa_jvp(rot(q), rot(k), v)`` for ``[B,S,H,D]`` tensors (views of a fused projection are
    fine), where ``rot`` is the rotary position embedding that semicat/net/duo.py:45-55 applies to q and
    k in front of the op, with fp32 ``cos``/``sin`` tables ``[S, D/2]``.  Where the kernels serve the
    shape (head dimension 64, at most 128 keys, bf16 / fp16 inputs with aligned rows) the rotation is
    folded into the attention launches: q and k are read unrotated, rotated on chip, and the gradients
    come back through the inverse rotation, so no rotary launch and no rotated copy of q, k exists in
    either AD mode.  Other shapes rotate with the library's rotary kernel first."""
    qh, kh, vh = q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2)
    tangents = [fwAD.unpack_dual(t).tangent for t in (qh, kh, vh)]
    if AUTOGRAD_WIRING != "reference" and kernels.rotary_fusable(
            fwAD.unpack_dual(qh).primal, fwAD.unpack_dual(kh).primal, cos,
            [fwAD.unpack_dual(vh).primal, *tangents], sin=sin):
        return _sdpa(qh, kh, vh, seq_major=True, cos=cos, sin=sin).transpose(1, 2)
    from .rotary import apply_rotary
    q, k = apply_rotary((q, k), cos, sin)
    return safe_sdpa_jvp(q, k, v)
