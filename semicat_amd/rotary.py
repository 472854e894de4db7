"""Rotary position embedding of q and k in front of the attention-JVP op, as one HIP launch with
both AD modes (``sjvp_rope`` in libsjvp.so).

The reference applies ``flash_attn.layers.rotary.apply_rotary_emb_torch`` to q and to k
(semicat/net/duo.py:45-55): separate fp32 PyTorch operations, followed by ``.contiguous()`` copies and
the cast to bf16 inside ``safe_sdpa_jvp`` (duo.py:141; jvp_utils/functional.py:318-322), each of them
once more for the forward-mode tangents.  The rotation is linear, so one kernel serves the primal,
the tangent (``jvp``) and, with the inverse rotation, the cotangent (``backward``); it reads the
``[B,S,H,D]`` slices of the fused qkv projection in place and writes contiguous 16-bit tensors that
the attention kernels take as they are.
"""
from __future__ import annotations

from typing import Optional

import torch
from torch import Tensor

from . import kernels


class RotaryFunction(torch.autograd.Function):
    """``y_i = R x_i`` for one to four tensors; ``R`` is orthogonal, so ``jvp`` is ``R t_i`` and
    ``backward`` is ``R^T g_i``, both through the same kernel.  ``out_dtype`` None keeps the input
    dtype; cotangents come back in the dtype of the inputs."""

    @staticmethod
    def forward(cos, sin, inverse, out_dtype, *xs):
        return kernels.rotary_embedding(xs, cos, sin, out_dtype=out_dtype, inverse=inverse)

    @staticmethod
    def setup_context(ctx, inputs, output):
        cos, sin, inverse, out_dtype, *xs = inputs
        ctx.save_for_backward(cos, sin)
        ctx.save_for_forward(cos, sin)
        ctx.inverse, ctx.out_dtype = inverse, out_dtype
        ctx.in_dtype = xs[0].dtype
        ctx.like = xs[0]
        ctx.set_materialize_grads(False)

    @staticmethod
    def jvp(ctx, _cos, _sin, _inverse, _out_dtype, *txs):
        cos, sin = ctx.saved_for_forward
        if all(t is None for t in txs):
            return tuple(None for _ in txs)
        txs = tuple(torch.zeros_like(ctx.like) if t is None else t for t in txs)
        return RotaryFunction.apply(cos, sin, ctx.inverse, ctx.out_dtype, *txs)

    @staticmethod
    def backward(ctx, *gs):
        cos, sin = ctx.saved_tensors
        present = [g for g in gs if g is not None]
        if not present:
            return (None,) * (4 + len(gs))
        outs = iter(RotaryFunction.apply(cos, sin, not ctx.inverse, ctx.in_dtype, *present))
        return (None, None, None, None, *[None if g is None else next(outs) for g in gs])


@torch._dynamo.disable
def apply_rotary(xs, cos: Tensor, sin: Tensor, out_dtype: Optional[torch.dtype] = None):
    """Rotate a tensor or a tuple of up to four ``[B,S,H,D]`` tensors (views are fine) by the fp32
    ``cos``/``sin`` tables ``[S, rot/2]``; returns contiguous ``[B,S,H,D]`` results."""
    single = isinstance(xs, Tensor)
    ys = RotaryFunction.apply(cos, sin, False, out_dtype, *((xs,) if single else tuple(xs)))
    return ys[0] if single else ys


@torch._dynamo.disable
def cast_tensors(xs, out_dtype: torch.dtype):
    """Cast a tensor or a tuple of up to four ``[B,S,H,D]`` tensors (views are fine) to ``out_dtype``
    in ONE launch, into contiguous ``[B,S,H,D]`` results: the rotary function without a rotation, so
    forward-mode tangents take the same launch and cotangents come back in the inputs' dtype through
    it.  This is the ``.to(torch.bfloat16)`` / ``.to(orig_dtype)`` pair that
    semicat/jvp_utils/functional.py:318-322,330-331 puts around the op for float32 callers."""
    single = isinstance(xs, Tensor)
    ys = RotaryFunction.apply(None, None, False, out_dtype, *((xs,) if single else tuple(xs)))
    return ys[0] if single else ys
