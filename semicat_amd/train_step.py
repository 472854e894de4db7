"""Losses of one semicat training step on a network with the ``net(x, s, t, jvp_attention=...)``
signature of :class:`semicat_amd.dit.DIT`, restated from olsdavis/semicat's
``semicat/models/semicat.py`` (cited by line below) without the Lightning module around them.

The self-distillation ("lag") loss is where the attention-JVP op earns its keep: it takes the
derivative of the flow map ``x_{s,t}`` with respect to the end time ``t`` by forward-mode AD over the
whole network and then back-propagates through that derivative (semicat.py:152-164).
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn


def _per_sample(t: Tensor, like: Tensor) -> Tensor:
    """``t`` ``[B]`` shaped to broadcast against ``like`` ``[B,...]`` (utils/shape.py:9-13)."""
    return t.reshape(like.shape[0], *([1] * (like.ndim - 1)))


def sample_prior(shape: tuple[int, ...], device, prior_type: str = "gaussian",
                 generator: Optional[torch.Generator] = None) -> Tensor:
    """Start point ``x0`` ``[B,S,V]``: standard normal, or a uniformly drawn one-hot
    (semicat.py:51-68)."""
    if prior_type == "gaussian":
        return torch.randn(shape, device=device, generator=generator)
    if prior_type == "discunif":
        cats = torch.randint(0, shape[-1], shape[:-1], device=device, generator=generator)
        return F.one_hot(cats, num_classes=shape[-1]).float()
    raise ValueError(f"unimplemented prior type `{prior_type}`")


def interpolate(x0: Tensor, x1: Tensor, t: Tensor) -> Tensor:
    """``(1 - t) x0 + t onehot(x1)`` with ``x1`` given as class indices (semicat.py:70-85)."""
    if x0.ndim != x1.ndim + 1 or t.ndim != x0.ndim:
        raise ValueError("x0 [B,S,V], x1 [B,S] (indices) and t [B,1,1] expected")
    xt = x0 * (1.0 - t)
    xt.scatter_add_(-1, x1.unsqueeze(-1), t.expand(*x1.shape, 1).to(xt.dtype))
    return xt


def flow_map(net: nn.Module, x: Tensor, s: Tensor, t: Tensor, jvp_attention: bool = False) -> Tensor:
    """``x_{s,t} = x + (t - s)/(1 - s) (softmax(net(x, s, t)) - x)`` (semicat.py:210-229)."""
    if s.shape != t.shape:
        raise ValueError("s and t must have the same shape")
    dt = (t - s) / (1.0 - s + 1e-8)
    target = net(x, s.reshape(-1), t.reshape(-1), jvp_attention=jvp_attention).softmax(dim=-1)
    return x + _per_sample(dt, x) * (target - x)


def vfm_loss(net: nn.Module, x0: Tensor, x1: Tensor, label_smoothing: float = 0.0,
             t: Optional[Tensor] = None) -> Tensor:
    """Cross-entropy of the end-point prediction at a random time (semicat.py:89-110)."""
    if t is None:
        t = torch.rand(x1.shape[0], device=x1.device)
    xt = interpolate(x0, x1, _per_sample(t, x0))
    logits = net(xt, t, t)
    # The reference writes F.cross_entropy(logits.transpose(-1, 1), x1) (semicat.py:106-110); with the
    # class axis moved away from the end PyTorch takes its strided softmax kernel, which needs tens
    # of milliseconds for a 30522-wide vocabulary.  The token-flattened form is the same mean over
    # all tokens with the class axis last.
    return F.cross_entropy(logits.reshape(-1, logits.shape[-1]), x1.reshape(-1),
                           label_smoothing=label_smoothing)


def lag_self_distillation_loss(net: nn.Module, x0: Tensor, x1: Tensor, t: Optional[Tensor] = None,
                               s: Optional[Tensor] = None) -> Tensor:
    """``mean_{b,s} sum_v ((1 - t) d/dt x_{s,t} - softmax(net(x_{s,t}, t, t)) + x_{s,t})^2`` with the
    time derivative by forward-mode AD through the network and gradients flowing through that
    derivative only (semicat.py:124-129, 152-164)."""
    B = x1.shape[0]
    if t is None:
        t = torch.rand(B, device=x1.device)
    if s is None:
        s = torch.rand(B, device=x1.device) * t
    xs = interpolate(x0, x1, _per_sample(s, x0))
    xst, dv = torch.func.jvp(lambda end: flow_map(net, xs, s, end, jvp_attention=True),
                             (t,), (torch.ones_like(t),))
    xst = xst.detach()
    with torch.no_grad():
        target = net(xst, t, t).softmax(dim=-1)
    return ((1.0 - _per_sample(t, xst)) * dv - target + xst).pow(2).sum(dim=-1).mean()


def model_step(net: nn.Module, x1: Tensor, in_shape: tuple[int, ...], sd_prop: float = 0.25,
               prior_type: str = "gaussian", label_smoothing: float = 0.0,
               generator: Optional[torch.Generator] = None) -> tuple[Tensor, Optional[Tensor]]:
    """The two losses of a step: the first ``int(sd_prop * B)`` samples take the self-distillation
    loss, the others the cross-entropy loss (semicat.py:169-191).  Returns ``(vfm, sd or None)``."""
    B = x1.shape[0]
    x0 = sample_prior((B, *in_shape), x1.device, prior_type, generator)
    split = int(sd_prop * B)
    vf = vfm_loss(net, x0[split:], x1[split:], label_smoothing)
    if split == 0:
        return vf, None
    return vf, lag_self_distillation_loss(net, x0[:split], x1[:split])


def compile_network(net: torch.nn.Module, backend: str = "aot_eager", **kwargs):
    """``torch.compile(net, backend=...)`` as the reference wraps its network (semicat.py:340-345), with
    the one backend that is known to fail here refused up front: on an MI355X box the reference's default,
    ``backend="inductor"``, once ended in a segmentation fault of the Python process while it compiled the
    PyTorch layers around the op (torch 2.10.0+rocm7.0, triton 3.6.0; cause not identified, not run
    again), so a network on a GPU is compiled with ``"aot_eager"`` (tested: both losses and the gradients
    equal the unwrapped network's) or left in eager mode.  On the CPU, inductor compiles the same
    network and matches eager.  The op itself is a graph break under every backend
    (``torch._dynamo.disable``, as functional.py:272)."""
    on_gpu = any(p.is_cuda for p in net.parameters())
    if backend == "inductor" and on_gpu:
        raise RuntimeError("backend='inductor' around a network on the GPU is not supported by this build: a run "
                           "on an MI355X box ended in a segmentation fault while inductor compiled the layers "
                           "around the op; use backend='aot_eager' or eager mode")
    return torch.compile(net, backend=backend, **kwargs)
