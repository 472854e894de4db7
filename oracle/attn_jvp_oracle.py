"""CPU oracle for the attention-JVP path.  TEST INFRASTRUCTURE ONLY.

Nothing here is part of the shipped product: only ``tests/``, ``__graft_entry__.smoke()`` and the
``cpu_baseline`` leg of ``bench.py`` may import this module.  The product path
(``semicat_amd``) never routes through it and has no CPU fallback.

What it restates (reference = olsdavis/semicat, paths relative to its root):

* ``attention_jvp_autograd``  - the reference's *math path*
  ``naive_multihead_attention_jvp`` (semicat/jvp_utils/ryu_triton.py:426-454):
  ``torch.func.jvp`` over eager ``softmax(Q K^T * scale) V``, evaluated in fp64, followed by
  ``torch.autograd.grad`` for the six input gradients given cotangents on O and on the tangent
  output.  This is the parity anchor.
* ``attention_jvp_closed_form`` - an independent numpy fp64 evaluation of the closed forms the
  reference's kernels implement: forward statistics M / MU / LI as defined at
  ryu_triton.py:271-291, ``dS_dot = P*(dTO V^T - sum_4)`` at flash_jvp_backward.py:251-257,
  ``dS`` at flash_jvp_backward.py:1364-1407 combined with the primal term ``P*(dO V^T - delta)`` of
  flash_attn_triton.py:606, ``P_dot = P*(S_dot - mu)`` at flash_jvp_backward.py:947-954 and the
  gradient contractions at :258-262, :592-601, :965-966, :1411-1416, :1841-1846.
* ``attention_jvp_online`` - the blocked online-softmax recurrence of the fused forward kernel
  (ryu_triton.py:188-291), including the row-statistic padding convention of
  functional.py:57-59,228-229 (rows >= L hold log(L_kv), 0, L_kv).
* ``attention_jvp_bruteforce`` - per-element Python loops, tiny shapes only.
* ``reference_rounding_error_model`` - the closed forms with the reference kernels' low-precision
  rounding points inserted (casts before every tl.dot: ryu_triton.py:241,255;
  flash_jvp_backward.py:240,257,590,596,951,966,1348,1409,1841), used to estimate the error the
  reference's own kernels would show against the fp64 math path on the same inputs.

Pinning status (tests/test_oracle.py): every function above is cross-checked against the others,
against central finite differences in fp64, against library routines (torch.logsumexp,
F.scaled_dot_product_attention autograd for the dTO = 0 special case), against invariants
(rows of P sum to 1, rows of P_dot sum to 0, linearity in the tangents, the q_dot = k_dot = 0
reduction to plain attention on V_dot) and against brute force.  The reference itself holds no
golden vectors for this path (its only test, ryu_triton.py:495-592, is a forward-only GPU script);
its five test shapes, seed, value scales and 1e-2 tolerance are reused in the tests.
"""
from __future__ import annotations

import math
from typing import Dict, Optional

import numpy as np
import torch

TENSOR_ORDER = ("q", "k", "v", "tq", "tk", "tv", "dO", "dTO")


def stat_rows(L: int) -> int:
    """Row-statistic length: L rounded up to 128 (ryu_triton.py:351, functional.py:57,228)."""
    return ((L + 127) // 128) * 128


def make_inputs(B: int, H: int, Lq: int, Lk: int, D: int, *, seed: int = 0,
                primal_scale: float = 1.0, tangent_scale: float = 1.0,
                dtype: torch.dtype = torch.float32) -> Dict[str, torch.Tensor]:
    """Seeded inputs: q,k,v,tq,tk,tv,dO,dTO drawn in this fixed order from one CPU generator as fp32
    N(0,1), then scaled, then cast to ``dtype``; layout [B,H,L,D] contiguous."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name in TENSOR_ORDER:
        L = Lk if name in ("k", "v", "tk", "tv") else Lq
        x = torch.randn(B, H, L, D, generator=g, dtype=torch.float32)
        if name in ("q", "k", "v"):
            x = x * primal_scale
        elif name in ("tq", "tk", "tv"):
            x = x * tangent_scale
        out[name] = x.to(dtype)
    return out


def _f64(x) -> torch.Tensor:
    return torch.as_tensor(x).detach().to(torch.float64).cpu()


def attention_math_path(q, k, v, scale):
    """softmax(Q K^T * scale) V - the function differentiated by the reference math path
    (ryu_triton.py:447-451)."""
    scores = torch.matmul(q, k.transpose(-2, -1)) * scale
    p = torch.softmax(scores, dim=-1)
    return torch.matmul(p, v)


def attention_jvp_autograd(q, k, v, tq, tk, tv, dO=None, dTO=None,
                           scale: Optional[float] = None,
                           dtype: torch.dtype = torch.float64) -> Dict[str, torch.Tensor]:
    """Reference math path in ``dtype`` (fp64 by default): O, TO via torch.func.jvp and, when a
    cotangent is given, the six gradients via torch.autograd.grad through the jvp graph."""
    q, k, v, tq, tk, tv = (torch.as_tensor(x).detach().to(dtype).cpu().clone().requires_grad_(True)
                           for x in (q, k, v, tq, tk, tv))
    D = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    O, TO = torch.func.jvp(lambda a, b, c: attention_math_path(a, b, c, scale),
                           (q, k, v), (tq, tk, tv))
    res = {"O": O.detach(), "TO": TO.detach()}
    if dO is None and dTO is None:
        return res
    outs, cots = [], []
    if dO is not None:
        outs.append(O)
        cots.append(torch.as_tensor(dO).detach().to(dtype).cpu())
    if dTO is not None:
        outs.append(TO)
        cots.append(torch.as_tensor(dTO).detach().to(dtype).cpu())
    grads = torch.autograd.grad(outs, [q, k, v, tq, tk, tv], cots, allow_unused=True)
    for name, g, ref in zip(("dq", "dk", "dv", "dtq", "dtk", "dtv"), grads,
                            (q, k, v, tq, tk, tv)):
        res[name] = torch.zeros_like(ref) if g is None else g.detach()
    return res


def attention_jvp_closed_form(q, k, v, tq, tk, tv, dO=None, dTO=None,
                              scale: Optional[float] = None) -> Dict[str, np.ndarray]:
    """Closed forms in numpy fp64.  Names follow the reference kernels' variables:
    sum_4 = rowsum(dTO*O), sum_7 = rowsum(dTO*TO), delta = rowsum(dO*O)."""
    q, k, v, tq, tk, tv = (_f64(x).numpy() for x in (q, k, v, tq, tk, tv))
    D = q.shape[-1]
    Lk = k.shape[-2]
    s = 1.0 / math.sqrt(D) if scale is None else float(scale)
    kT = np.swapaxes(k, -1, -2)
    tkT = np.swapaxes(tk, -1, -2)
    S = s * (q @ kT)
    m = S.max(-1, keepdims=True)
    E = np.exp(S - m)
    l = E.sum(-1, keepdims=True)
    P = E / l
    lse = (m + np.log(l))[..., 0]
    TS = s * (tq @ kT + q @ tkT)
    mu = (P * TS).sum(-1, keepdims=True)
    N = TS - mu
    PD = P * N
    O = P @ v
    TO = PD @ v + P @ tv
    res = {"O": O, "TO": TO, "lse": lse, "mu": mu[..., 0], "li": l[..., 0], "Lk": Lk}
    if dO is None and dTO is None:
        return res
    G = np.zeros_like(O) if dTO is None else _f64(dTO).numpy()
    dOn = np.zeros_like(O) if dO is None else _f64(dO).numpy()
    vT = np.swapaxes(v, -1, -2)
    tvT = np.swapaxes(tv, -1, -2)
    sum_4 = (G * O).sum(-1, keepdims=True)
    sum_7 = (G * TO).sum(-1, keepdims=True)
    delta = (dOn * O).sum(-1, keepdims=True)
    W = G @ vT
    X = G @ tvT
    Y = dOn @ vT
    dTS = P * (W - sum_4)
    dS = dTS * N + P * (X + Y - sum_7 - delta)
    dTSt = np.swapaxes(dTS, -1, -2)
    dSt = np.swapaxes(dS, -1, -2)
    res.update(
        dtq=s * (dTS @ k),
        dtk=s * (dTSt @ q),
        dtv=np.swapaxes(P, -1, -2) @ G,
        dq=s * (dS @ k + dTS @ tk),
        dk=s * (dSt @ q + dTSt @ tq),
        dv=np.swapaxes(PD, -1, -2) @ G + np.swapaxes(P, -1, -2) @ dOn,
        sum_4=sum_4[..., 0], sum_7=sum_7[..., 0], delta=delta[..., 0],
    )
    return res


def attention_jvp_online(q, k, v, tq, tk, tv, scale: Optional[float] = None,
                         block_m: int = 64, block_n: int = 32) -> Dict[str, np.ndarray]:
    """The fused forward kernel's online recurrence (ryu_triton.py:188-291) in numpy fp64, block by
    block, including the statistics buffers M / MU / LI of length stat_rows(L) whose rows >= L keep
    their initial values log(L_kv), 0, L_kv (functional.py:57-59,228-229)."""
    q, k, v, tq, tk, tv = (_f64(x).numpy() for x in (q, k, v, tq, tk, tv))
    B, H, L, D = q.shape
    Lk = k.shape[-2]
    s = 1.0 / math.sqrt(D) if scale is None else float(scale)
    Lr = stat_rows(L)
    O = np.zeros((B, H, L, D))
    TO = np.zeros((B, H, L, D))
    M = np.full((B, H, Lr), math.log(Lk))
    MU = np.zeros((B, H, Lr))
    LI = np.full((B, H, Lr), float(Lk))
    for b in range(B):
        for h in range(H):
            for m0 in range(0, L, block_m):
                rows = slice(m0, min(m0 + block_m, L))
                qb, tqb = q[b, h, rows], tq[b, h, rows]
                nr = qb.shape[0]
                m_i = np.full(nr, -np.inf)
                l_i = np.ones(nr)            # ryu_triton.py:189 (the "+1" is wiped by alpha = 0)
                mu_i = np.zeros(nr)
                acc = np.zeros((nr, D))
                g_acc = np.zeros((nr, D))
                ptv = np.zeros((nr, D))
                for n0 in range(0, Lk, block_n):
                    cols = slice(n0, min(n0 + block_n, Lk))
                    kb, vb, tkb, tvb = k[b, h, cols], v[b, h, cols], tk[b, h, cols], tv[b, h, cols]
                    qk = qb @ kb.T
                    tqk = tqb @ kb.T + qb @ tkb.T
                    m_ij = np.maximum(m_i, (qk * s).max(1))
                    p = np.exp(qk * s - m_ij[:, None])
                    alpha = np.exp(m_i - m_ij)
                    l_i = l_i * alpha + p.sum(1)
                    acc = acc * alpha[:, None] + p @ vb
                    p_tqk = p * (tqk * s)
                    mu_i = mu_i * alpha + p_tqk.sum(1)
                    g_acc = g_acc * alpha[:, None] + p_tqk @ vb
                    ptv = ptv * alpha[:, None] + p @ tvb
                    m_i = m_ij
                y = acc / l_i[:, None]
                O[b, h, rows] = y
                TO[b, h, rows] = (g_acc - mu_i[:, None] * y + ptv) / l_i[:, None]
                M[b, h, rows] = m_i + np.log(l_i)
                MU[b, h, rows] = mu_i / l_i
                LI[b, h, rows] = l_i
    return {"O": O, "TO": TO, "M": M, "MU": MU, "LI": LI}


def attention_jvp_bruteforce(q, k, v, tq, tk, tv, dO, dTO, scale: Optional[float] = None):
    """Per-element loops on [L,D] python lists (one (b,h) slice); the gradients are obtained by
    accumulating, element by element, the chain rule through
    S -> P -> (O, TO) written out from the definitions, with no matrix algebra shared with the
    closed-form routine.  Tiny shapes only."""
    q, k, v, tq, tk, tv, dO, dTO = (_f64(x).numpy() for x in (q, k, v, tq, tk, tv, dO, dTO))
    assert q.ndim == 2
    L, D = q.shape
    Lk = k.shape[0]
    s = 1.0 / math.sqrt(D) if scale is None else float(scale)
    O = [[0.0] * D for _ in range(L)]
    TO = [[0.0] * D for _ in range(L)]
    dq = [[0.0] * D for _ in range(L)]
    dtq = [[0.0] * D for _ in range(L)]
    dk = [[0.0] * D for _ in range(Lk)]
    dtk = [[0.0] * D for _ in range(Lk)]
    dv = [[0.0] * D for _ in range(Lk)]
    dtv = [[0.0] * D for _ in range(Lk)]
    for i in range(L):
        sc = [s * sum(q[i][d] * k[j][d] for d in range(D)) for j in range(Lk)]
        tsc = [s * sum(tq[i][d] * k[j][d] + q[i][d] * tk[j][d] for d in range(D))
               for j in range(Lk)]
        mx = max(sc)
        e = [math.exp(x - mx) for x in sc]
        z = sum(e)
        p = [x / z for x in e]
        mu = sum(p[j] * tsc[j] for j in range(Lk))
        pd = [p[j] * (tsc[j] - mu) for j in range(Lk)]
        for d in range(D):
            O[i][d] = sum(p[j] * v[j][d] for j in range(Lk))
            TO[i][d] = sum(pd[j] * v[j][d] + p[j] * tv[j][d] for j in range(Lk))
        # cotangents on p_j and pd_j
        gp = [sum(dO[i][d] * v[j][d] + dTO[i][d] * tv[j][d] for d in range(D)) for j in range(Lk)]
        gpd = [sum(dTO[i][d] * v[j][d] for d in range(D)) for j in range(Lk)]
        for j in range(Lk):
            for d in range(D):
                dv[j][d] += p[j] * dO[i][d] + pd[j] * dTO[i][d]
                dtv[j][d] += p[j] * dTO[i][d]
        # pd_j = p_j (tsc_j - mu),  mu = sum_j p_j tsc_j
        gmu = -sum(gpd[j] * p[j] for j in range(Lk))
        gtsc = [gpd[j] * p[j] + gmu * p[j] for j in range(Lk)]
        gp_tot = [gp[j] + gpd[j] * (tsc[j] - mu) + gmu * tsc[j] for j in range(Lk)]
        # p = softmax(sc)
        dot = sum(gp_tot[j] * p[j] for j in range(Lk))
        gsc = [p[j] * (gp_tot[j] - dot) for j in range(Lk)]
        for j in range(Lk):
            for d in range(D):
                dq[i][d] += s * (gsc[j] * k[j][d] + gtsc[j] * tk[j][d])
                dtq[i][d] += s * gtsc[j] * k[j][d]
                dk[j][d] += s * (gsc[j] * q[i][d] + gtsc[j] * tq[i][d])
                dtk[j][d] += s * gtsc[j] * q[i][d]
    return {n: np.array(x) for n, x in dict(O=O, TO=TO, dq=dq, dk=dk, dv=dv, dtq=dtq, dtk=dtk,
                                            dtv=dtv).items()}


def _round_to(x: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    return torch.from_numpy(np.ascontiguousarray(x)).to(dtype).to(torch.float64).numpy()


def reference_rounding_error_model(q, k, v, tq, tk, tv, dO, dTO, dtype=torch.bfloat16,
                                   scale: Optional[float] = None) -> Dict[str, np.ndarray]:
    """Closed forms with the reference kernels' rounding points: inputs already in ``dtype``;
    the probability tile, the tangent-weighted tile and every gradient tile are rounded to
    ``dtype`` before they enter a contraction; accumulation is exact (fp64 here, fp32 there);
    outputs are rounded to ``dtype``; the partial dq / dk written by the first backward kernels are
    rounded to ``dtype`` before the second kernels add to them (functional.py:115-116 with
    flash_jvp_backward.py:1196,1641).  The two cotangent paths are evaluated separately and summed in
    ``dtype`` as autograd would."""
    r = lambda x: _round_to(x, dtype)
    q, k, v, tq, tk, tv, dOn, G = (r(_f64(x).numpy()) for x in (q, k, v, tq, tk, tv, dO, dTO))
    D = q.shape[-1]
    s = 1.0 / math.sqrt(D) if scale is None else float(scale)
    T = lambda x: np.swapaxes(x, -1, -2)
    S = s * (q @ T(k))
    m = S.max(-1, keepdims=True)
    E = np.exp(S - m)
    l = E.sum(-1, keepdims=True)
    TS = s * (tq @ T(k) + q @ T(tk))
    Et = r(E)
    ETS = E * TS
    mu_un = ETS.sum(-1, keepdims=True)
    acc = Et @ v
    g_acc = r(ETS) @ v
    ptv = Et @ tv
    y = acc / l
    O = r(y)
    TO = r((g_acc - mu_un * y + ptv) / l)
    mu = mu_un / l
    lse = m + np.log(l)
    P = np.exp(S - lse)
    Pt = r(P)
    N = TS - mu
    # cotangent on the tangent output (flash_jvp_backward.py)
    sum_4 = (Pt * (G @ T(v))).sum(-1, keepdims=True)
    sum_7 = (Pt * ((G @ T(v)) * N + G @ T(tv))).sum(-1, keepdims=True)
    W = G @ T(v)
    dTS = r(Pt * (W - sum_4) * s)
    dtk = r(T(dTS) @ q)
    dk_part = r(T(dTS) @ tq)
    dtq = r(dTS @ k)
    dq_part = r(dTS @ tk)
    PD = r(P * N)
    dtv = r(T(Pt) @ G)
    dv_j = r(T(PD) @ G)
    mul_8 = -sum_4 * (P * N)
    fma = (G @ T(tv) + W * N - sum_7) * Pt
    dSj = r((mul_8 + fma) * s)
    dk_j = r(dk_part + r(T(dSj) @ q))
    dq_j = r(dq_part + r(dSj @ k))
    # cotangent on the primal output (flash_attn_triton.py:526-617)
    delta = (O * dOn).sum(-1, keepdims=True)
    dv_p = r(T(Pt) @ dOn)
    dSp = r(P * (dOn @ T(v) - delta) * s)
    dk_p = r(T(dSp) @ q)
    dq_p = r(dSp @ k)
    return {"O": O, "TO": TO, "dq": r(dq_j + dq_p), "dk": r(dk_j + dk_p), "dv": r(dv_j + dv_p),
            "dtq": dtq, "dtk": dtk, "dtv": dtv}


def row_sum_rounding_model(q, k, v, tq, tk, tv, dO, dTO, dtype=torch.bfloat16, sums_from_outputs=True,
                           scale: Optional[float] = None, repaired: bool = False) -> Dict[str, np.ndarray]:
    """The query-side and key-side gradients with the two row sums of the backward formed either from
    the outputs rounded to ``dtype`` (``s4 = rowsum(G*O)``, ``s7d = rowsum(G*TO) + rowsum(dO*O)``: the
    FlashAttention "delta" form, extended to the cotangent on the tangent output) or from the
    probabilities themselves (``rowsum(P*W)``, ``rowsum(P*(N*W + XY))``, what the reference's preprocess
    kernel does, flash_jvp_backward.py:2012-2290); everything else exact up to one rounding of the
    score-gradient tiles and of the results.  ``sum_j P (W - s4) = 0`` holds exactly only in the second
    form; in the first the rounding of O leaves a residue that is the same for every key of a row and
    so adds up coherently in ``dS_dot^T Q`` and ``dS_dot K``.

    ``repaired`` (with ``sums_from_outputs``) models what the row-owned + column-owned kernels do about
    it: the residues ``rho4 = sum_j dS_dot``, ``rho7 = sum_j dS`` (zero with exact sums) are measured on
    the unrounded tiles formed with the rounded sums, and every gradient is then formed with the
    corrected sums ``s4 + rho4``, ``s7d + rho7`` (the column pass always, the row pass in its second
    launch).  In exact arithmetic the corrected sums are the sums of the second form.
    Returns dq, dk, dtq, dtk."""
    r = lambda x: _round_to(x, dtype)
    q, k, v, tq, tk, tv, dOn, G = (r(_f64(x).numpy()) for x in (q, k, v, tq, tk, tv, dO, dTO))
    s = 1.0 / math.sqrt(q.shape[-1]) if scale is None else float(scale)
    T = lambda x: np.swapaxes(x, -1, -2)
    S = s * (q @ T(k))
    E = np.exp(S - S.max(-1, keepdims=True))
    P = E / E.sum(-1, keepdims=True)
    TS = s * (tq @ T(k) + q @ T(tk))
    N = TS - (P * TS).sum(-1, keepdims=True)
    O, TO = r(P @ v), r((P * N) @ v + P @ tv)
    W, XY = G @ T(v), G @ T(tv) + dOn @ T(v)
    if sums_from_outputs:
        s4 = (G * O).sum(-1, keepdims=True)
        s7d = (G * TO).sum(-1, keepdims=True) + (dOn * O).sum(-1, keepdims=True)
    else:
        s4 = (P * W).sum(-1, keepdims=True)
        s7d = (P * (N * W + XY)).sum(-1, keepdims=True)
    dTS = P * (W - s4)
    dS = dTS * N + P * (XY - s7d)
    if repaired and sums_from_outputs:
        s4 = s4 + dTS.sum(-1, keepdims=True)
        s7d = s7d + dS.sum(-1, keepdims=True)
        dTS = P * (W - s4)
        dS = dTS * N + P * (XY - s7d)
    dS = r(dS)
    dTS = r(dTS)
    return {"dq": r(s * (dS @ k + dTS @ tk)), "dk": r(s * (T(dS) @ q + T(dTS) @ tq)),
            "dtq": r(s * dTS @ k), "dtk": r(s * T(dTS) @ q)}


def rel_frobenius(x, ref) -> float:
    """||x - ref||_F / ||ref||_F in fp64 (the accuracy gate's measure)."""
    x = _f64(x)
    ref = _f64(ref)
    den = float(torch.linalg.vector_norm(ref))
    num = float(torch.linalg.vector_norm(x - ref))
    return num / den if den > 0 else num
