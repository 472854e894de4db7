"""Eager-torch stand-ins for the three kernel launchers in semicat_amd.kernels, used ONLY by the
CPU tests of the host-side autograd wiring (monkeypatched in; never shipped, never a fallback).
They honour the same in-place output contract as the HIP launchers."""
import math

import torch

from semicat_amd.kernels import stat_rows


def _stats(S, TS, Lq, Lk):
    B, H = S.shape[:2]
    Lr = stat_rows(Lq)
    lse = torch.full((B, H, Lr), math.log(Lk), dtype=torch.float32)
    mu = torch.zeros((B, H, Lr), dtype=torch.float32)
    lse[..., :Lq] = torch.logsumexp(S, -1)
    if TS is not None:
        mu[..., :Lq] = (torch.softmax(S, -1) * TS).sum(-1)
    return lse, mu


def _reader(arithmetic):
    """How a launcher sees its inputs: as fp32 values, rounded to bf16 first with arithmetic="bf16"."""
    if arithmetic == "bf16":
        return lambda t: None if t is None else t.detach().to(torch.bfloat16).float()
    return lambda t: None if t is None else t.detach().float()


def _rot(x, rope, inverse=False):
    """Rotary embedding of a [B,H,L,D] tensor by (cos, sin) [L, D/2] tables; x unchanged without rope."""
    if rope is None or x is None:
        return x
    cos, sin = (t[: x.shape[-2]].float() for t in rope)
    if inverse:
        sin = -sin
    half = cos.shape[-1]
    x1, x2 = x[..., :half], x[..., half:2 * half]
    return torch.cat((x1 * cos - x2 * sin, x2 * cos + x1 * sin, x[..., 2 * half:]), dim=-1)


def attention_jvp_forward(q, k, v, tq, tk, tv, scale=None, o=None, to=None, lse=None, mu=None,
                          li=None, with_li=True, arithmetic=None, rope=None):
    f = _reader(arithmetic)
    qf, kf, vf, tqf, tkf, tvf = map(f, (q, k, v, tq, tk, tv))
    qf, kf, tqf, tkf = (_rot(t, rope) for t in (qf, kf, tqf, tkf))
    s = scale or 1.0 / math.sqrt(q.shape[-1])
    S = s * qf @ kf.transpose(-1, -2)
    TS = s * (tqf @ kf.transpose(-1, -2) + qf @ tkf.transpose(-1, -2))
    P = torch.softmax(S, -1)
    mu_ = (P * TS).sum(-1, keepdim=True)
    O = P @ vf
    TO = (P * (TS - mu_)) @ vf + P @ tvf
    lse_, mu_full = _stats(S, TS, q.shape[-2], k.shape[-2])
    o = torch.empty_like(q) if o is None else o
    to = torch.empty_like(q) if to is None else to
    # .data: like a raw kernel launch, the write does not bump the autograd version counter
    o.data.copy_(O)
    to.data.copy_(TO)
    if lse is None:
        lse = lse_
    else:
        lse.data.copy_(lse_)
    if mu is None:
        mu = mu_full
    else:
        mu.data.copy_(mu_full)
    return o, to, lse, mu, None


def attention_forward(q, k, v, scale=None, o=None, lse=None, arithmetic=None, rope=None):
    f = _reader(arithmetic)
    s = scale or 1.0 / math.sqrt(q.shape[-1])
    S = s * _rot(f(q), rope) @ _rot(f(k), rope).transpose(-1, -2)
    O = torch.softmax(S, -1) @ f(v)
    lse_, _ = _stats(S, None, q.shape[-2], k.shape[-2])
    o = torch.empty_like(q) if o is None else o
    o.data.copy_(O)
    if lse is None:
        lse = lse_
    else:
        lse.data.copy_(lse_)
    return o, lse


def attention_jvp_backward(q, k, v, tq, tk, tv, o, to, lse, mu, dO=None, dTO=None, scale=None,
                           grads=None, arithmetic=None, rope=None):
    assert dO is not None or dTO is not None
    f = _reader(arithmetic)
    Lq = q.shape[-2]
    s = scale or 1.0 / math.sqrt(q.shape[-1])
    qf, kf, vf, of = _rot(f(q), rope), _rot(f(k), rope), f(v), f(o)
    T = lambda x: x.transpose(-1, -2)
    P = torch.exp(s * qf @ T(kf) - lse[..., :Lq, None])
    z = torch.zeros_like(of)
    dOf = z if dO is None else f(dO)
    if dTO is None:
        dS = P * (dOf @ T(vf) - (dOf * of).sum(-1, keepdim=True))
        out = (s * dS @ kf, s * T(dS) @ qf, T(P) @ dOf, None, None, None)
    else:
        tqf, tkf, tvf, tof, G = _rot(f(tq), rope), _rot(f(tk), rope), f(tv), f(to), f(dTO)
        N = s * (tqf @ T(kf) + qf @ T(tkf)) - mu[..., :Lq, None]
        s4 = (G * of).sum(-1, keepdim=True)
        s7d = (G * tof).sum(-1, keepdim=True) + (dOf * of).sum(-1, keepdim=True)
        dTS = P * (G @ T(vf) - s4)
        dS = dTS * N + P * (G @ T(tvf) + dOf @ T(vf) - s7d)
        out = (s * (dS @ kf + dTS @ tkf), s * (T(dS) @ qf + T(dTS) @ tqf), T(P * N) @ G + T(P) @ dOf,
               s * dTS @ kf, s * T(dTS) @ qf, T(P) @ G)
    # gradients of rotated tensors go back through the inverse rotation
    out = tuple(_rot(g, rope, inverse=True) if i in (0, 1, 3, 4) else g for i, g in enumerate(out))
    if grads is None:
        like = (q, k, v, tq, tk, tv)
        return tuple(None if g is None else g.to(l.dtype) for g, l in zip(out, like))
    for dst, g in zip(grads, out):
        if dst is not None and g is not None:
            dst.data.copy_(g)
    return grads


def install(monkeypatch):
    import semicat_amd.kernels as K
    monkeypatch.setattr(K, "attention_jvp_forward", attention_jvp_forward)
    monkeypatch.setattr(K, "attention_forward", attention_forward)
    monkeypatch.setattr(K, "attention_jvp_backward", attention_jvp_backward)
