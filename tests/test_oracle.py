"""Pins the CPU oracle (oracle/) without the reference: the autograd math path, the numpy closed
forms, the C restatement, the online recurrence and brute force must agree with each other, with
finite differences, with library routines and with the invariants of the mathematics."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import attn_jvp_oracle as orc
from oracle import c_ref

GRADS = ("dq", "dk", "dv", "dtq", "dtk", "dtv")
# the reference's own test shapes and scales (ryu_triton.py:504-524): (B,H,L,D), seed 42,
# N(0,1) primals, tangents * 0.1
REF_SHAPES = [(1, 1, 8, 16), (2, 2, 16, 32), (1, 4, 32, 32), (1, 1, 64, 64), (2, 3, 128, 16)]


def _inputs(shape, Lk=None, seed=42, dtype=torch.float64, ts=0.1):
    B, H, L, D = shape
    return orc.make_inputs(B, H, L, Lk or L, D, seed=seed, tangent_scale=ts, dtype=dtype)


def _args(x):
    return [x[n] for n in orc.TENSOR_ORDER]


@pytest.mark.parametrize("shape", REF_SHAPES)
def test_closed_form_matches_autograd(shape):
    x = _inputs(shape)
    a = orc.attention_jvp_autograd(*_args(x))
    c = orc.attention_jvp_closed_form(*_args(x))
    for n in ("O", "TO") + GRADS:
        assert orc.rel_frobenius(c[n], a[n]) < 1e-12, n


@pytest.mark.parametrize("shape,Lk", [((1, 2, 8, 16), 8), ((2, 1, 37, 16), 53), ((1, 1, 130, 32), 70)])
def test_c_restatement_matches_autograd(shape, Lk):
    x = _inputs(shape, Lk=Lk)
    a = orc.attention_jvp_autograd(*_args(x))
    c = c_ref.attention_jvp_c(*_args(x))
    for n in ("O", "TO") + GRADS:
        assert orc.rel_frobenius(c[n], a[n]) < 1e-12, n
    cf = orc.attention_jvp_closed_form(*_args(x))
    L = shape[2]
    np.testing.assert_allclose(c["M"][..., :L], cf["lse"], rtol=1e-12)
    np.testing.assert_allclose(c["MU"][..., :L], cf["mu"], rtol=1e-10, atol=1e-13)
    np.testing.assert_allclose(c["LI"][..., :L], cf["li"], rtol=1e-12)
    # padded statistic rows keep log(Lk), 0, Lk
    assert np.all(c["M"][..., L:] == math.log(Lk))
    assert np.all(c["MU"][..., L:] == 0.0)
    assert np.all(c["LI"][..., L:] == Lk)


def test_c_restatement_single_cotangent():
    x = _inputs((1, 2, 9, 16), Lk=11)
    a = _args(x)
    for keep in ("dO", "dTO"):
        kw = dict(dO=x["dO"] if keep == "dO" else None, dTO=x["dTO"] if keep == "dTO" else None)
        ag = orc.attention_jvp_autograd(*a[:6], **kw)
        c = c_ref.attention_jvp_c(*a[:6], **kw)
        for n in GRADS:
            assert orc.rel_frobenius(c[n], ag[n]) < 1e-12 or np.abs(c[n]).max() == 0, n


def test_bruteforce_matches_autograd():
    x = _inputs((1, 1, 5, 16), Lk=7, ts=1.0)
    a = orc.attention_jvp_autograd(*_args(x))
    b = orc.attention_jvp_bruteforce(*[t[0, 0] for t in _args(x)])
    for n in ("O", "TO") + GRADS:
        assert orc.rel_frobenius(b[n], a[n][0, 0]) < 1e-12, n


@pytest.mark.parametrize("bm,bn", [(64, 32), (16, 8), (7, 5)])
def test_online_recurrence_matches_closed_form(bm, bn):
    x = _inputs((2, 2, 45, 16), Lk=39, ts=1.0)
    a = _args(x)[:6]
    on = orc.attention_jvp_online(*a, block_m=bm, block_n=bn)
    cf = orc.attention_jvp_closed_form(*a)
    L, Lk = 45, 39
    np.testing.assert_allclose(on["O"], cf["O"], rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(on["TO"], cf["TO"], rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(on["M"][..., :L], cf["lse"], rtol=1e-12)
    np.testing.assert_allclose(on["MU"][..., :L], cf["mu"], rtol=1e-10, atol=1e-13)
    assert on["M"].shape[-1] == 128
    assert np.all(on["M"][..., L:] == math.log(Lk)) and np.all(on["LI"][..., L:] == Lk)
    # LI is the exp-sum relative to the row max: lse = max + log(LI)
    S = (x["q"] @ x["k"].transpose(-1, -2)).numpy() / math.sqrt(16)
    np.testing.assert_allclose(on["LI"][..., :L], np.exp(S - S.max(-1, keepdims=True)).sum(-1),
                               rtol=1e-12)


def test_forward_against_library_routines():
    x = _inputs((2, 3, 33, 32), Lk=41)
    cf = orc.attention_jvp_closed_form(*_args(x)[:6])
    S = (x["q"] @ x["k"].transpose(-1, -2)) / math.sqrt(32)
    np.testing.assert_allclose(cf["lse"], torch.logsumexp(S, -1).numpy(), rtol=1e-13)
    O = F.scaled_dot_product_attention(x["q"], x["k"], x["v"])
    assert orc.rel_frobenius(cf["O"], O) < 1e-13


def test_tangent_against_finite_difference():
    x = _inputs((1, 2, 19, 16), Lk=23, ts=1.0)
    q, k, v, tq, tk, tv = _args(x)[:6]
    a = orc.attention_jvp_autograd(q, k, v, tq, tk, tv)
    eps = 1e-6
    s = 1 / math.sqrt(16)
    fp = orc.attention_math_path(q + eps * tq, k + eps * tk, v + eps * tv, s)
    fm = orc.attention_math_path(q - eps * tq, k - eps * tk, v - eps * tv, s)
    assert orc.rel_frobenius(a["TO"], (fp - fm) / (2 * eps)) < 1e-8


def test_gradients_against_finite_difference():
    """<dO,O> + <dTO,TO> as a scalar function of the six inputs: directional derivative along a
    random direction must equal the inner product of the gradients with that direction."""
    x = _inputs((1, 1, 11, 16), Lk=13, ts=1.0)
    a = _args(x)
    res = orc.attention_jvp_closed_form(*a)
    g = torch.Generator().manual_seed(7)
    dirs = [torch.randn(t.shape, generator=g, dtype=torch.float64) for t in a[:6]]

    def phi(inp):
        r = orc.attention_jvp_closed_form(*inp)
        return float((r["O"] * a[6].numpy()).sum() + (r["TO"] * a[7].numpy()).sum())

    eps = 1e-6
    plus = [t + eps * d for t, d in zip(a[:6], dirs)]
    minus = [t - eps * d for t, d in zip(a[:6], dirs)]
    fd = (phi(plus) - phi(minus)) / (2 * eps)
    an = sum(float((res[n] * d.numpy()).sum()) for n, d in zip(GRADS, dirs))
    assert abs(fd - an) < 1e-7 * max(1.0, abs(an))


def test_invariants():
    x = _inputs((2, 2, 17, 16), Lk=29, ts=1.0)
    q, k, v, tq, tk, tv, dO, dTO = _args(x)
    # constant V: O = const and the P_dot V part vanishes (rows of P_dot sum to zero)
    vc = torch.ones_like(v) * 0.37
    r = orc.attention_jvp_closed_form(q, k, vc, tq, tk, torch.zeros_like(tv))
    np.testing.assert_allclose(r["O"], 0.37, rtol=1e-13)
    assert np.abs(r["TO"]).max() < 1e-14
    # q_dot = k_dot = 0: the tangent is plain attention on V_dot
    z = torch.zeros_like
    r = orc.attention_jvp_closed_form(q, k, v, z(tq), z(tk), tv)
    assert orc.rel_frobenius(r["TO"], F.scaled_dot_product_attention(q, k, tv)) < 1e-13
    # linearity in the tangents
    r1 = orc.attention_jvp_closed_form(q, k, v, tq, tk, tv)
    r2 = orc.attention_jvp_closed_form(q, k, v, 2 * tq, 2 * tk, 2 * tv)
    assert orc.rel_frobenius(r2["TO"], 2 * r1["TO"]) < 1e-13
    # dTO = 0: standard attention backward from the library's autograd
    qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(qq, kk, vv).backward(dO)
    r = orc.attention_jvp_closed_form(q, k, v, tq, tk, tv, dO=dO, dTO=None)
    for n, t in (("dq", qq), ("dk", kk), ("dv", vv)):
        assert orc.rel_frobenius(r[n], t.grad) < 1e-12, n
    for n in ("dtq", "dtk", "dtv"):
        assert np.abs(r[n]).max() == 0
    # dO = 0 and q_dot = k_dot = 0: dV_dot = P^T dTO and dV = 0
    r = orc.attention_jvp_closed_form(q, k, v, z(tq), z(tk), tv, dO=None, dTO=dTO)
    P = torch.softmax((q @ k.transpose(-1, -2)) / 4.0, -1)
    assert orc.rel_frobenius(r["dtv"], P.transpose(-1, -2) @ dTO) < 1e-13
    assert np.abs(r["dv"]).max() < 1e-13


def test_temperature_derivative():
    """k_dot = v_dot = 0, q_dot = c*q: the tangent is c * d/dtau softmax(tau S) V at tau = 1."""
    x = _inputs((1, 1, 9, 16), Lk=12)
    q, k, v = x["q"], x["k"], x["v"]
    c = 0.3
    r = orc.attention_jvp_closed_form(q, k, v, c * q, torch.zeros_like(k), torch.zeros_like(v))
    eps = 1e-6
    s = 1 / 4.0
    fd = (orc.attention_math_path(q, k, v, s * (1 + eps)) -
          orc.attention_math_path(q, k, v, s * (1 - eps))) / (2 * eps)
    assert orc.rel_frobenius(r["TO"], c * fd) < 1e-8


def test_fp32_math_path_meets_1e5_bound():
    """Config 1 (B=2,H=4,L=256,D=64, fp32, seed 0): the fp32 CPU math path stays within 1e-5
    relative Frobenius of its fp64 evaluation on all eight outputs."""
    x = orc.make_inputs(2, 4, 256, 256, 64, seed=0, dtype=torch.float32)
    a64 = orc.attention_jvp_autograd(*_args(x))
    a32 = orc.attention_jvp_autograd(*_args(x), dtype=torch.float32)
    for n in ("O", "TO") + GRADS:
        assert orc.rel_frobenius(a32[n], a64[n]) < 1e-5, n


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_reference_rounding_model_is_within_authors_tolerance(dtype):
    """The emulated reference rounding stays inside the 1e-2 the reference's authors accept
    (ryu_triton.py:551-554) on the forward outputs and is self-consistent on the gradients."""
    x = orc.make_inputs(2, 2, 64, 64, 32, seed=42, tangent_scale=0.1, dtype=dtype)
    a = orc.attention_jvp_autograd(*_args(x))
    m = orc.reference_rounding_error_model(*_args(x), dtype=dtype)
    for n in ("O", "TO") + GRADS:
        assert orc.rel_frobenius(m[n], a[n]) < 2e-2, n
    m64 = orc.reference_rounding_error_model(*_args(x), dtype=torch.float64)
    for n in ("O", "TO") + GRADS:
        assert orc.rel_frobenius(m64[n], a[n]) < 1e-12, n


def test_row_sums_from_rounded_outputs_leave_a_coherent_residue():
    """The row-sum model: with the sums taken from the probabilities the gradients carry the error of
    one rounding (a few 1e-3 in bf16); with the sums taken from the rounded outputs, as the HIP kernels
    and every FlashAttention-style backward take them, a row whose `sum_j P (W - s4)` cancels strongly
    shows several times that (two query rows, 255 keys, logits of scale 2: 1.4e-2 on dq_dot, dk_dot).
    Both forms agree with the fp64 gradients to their own accuracy on an ordinary shape."""
    x = orc.make_inputs(2, 1, 2, 255, 40, seed=1062, primal_scale=2.0, tangent_scale=0.3, dtype=torch.bfloat16)
    ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
    args = [x[n] for n in orc.TENSOR_ORDER]
    exact = orc.row_sum_rounding_model(*args, sums_from_outputs=False)
    delta = orc.row_sum_rounding_model(*args, sums_from_outputs=True)
    e_exact = {n: orc.rel_frobenius(torch.from_numpy(v), ref[n]) for n, v in exact.items()}
    e_delta = {n: orc.rel_frobenius(torch.from_numpy(v), ref[n]) for n, v in delta.items()}
    assert max(e_exact.values()) <= 5e-3, e_exact
    assert e_delta["dtq"] >= 3 * e_exact["dtq"] and e_delta["dtk"] >= 3 * e_exact["dtk"], (e_exact, e_delta)
    assert max(e_delta.values()) <= 2.5e-2, e_delta
    x = orc.make_inputs(2, 2, 64, 64, 32, seed=7, tangent_scale=0.3, dtype=torch.bfloat16)
    ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
    for form in (False, True):
        m = orc.row_sum_rounding_model(*[x[n] for n in orc.TENSOR_ORDER], sums_from_outputs=form)
        assert max(orc.rel_frobenius(torch.from_numpy(v), ref[n]) for n, v in m.items()) <= 6e-3


def test_repaired_row_sums_match_the_sums_from_the_probabilities():
    """The repaired form of the row-sum model (residues of dS_dot, dS summed over the keys and added to
    the sums, every gradient formed again with the corrected sums) is as accurate as the reference's
    form on the cases where the sums of the rounded outputs alone fail: the 255-key case,
    a saturated single row in fp16 (0.9998 of the probability on one of five keys: 0.5-0.6 relative
    error without the repair) and constructed saturated rows in bf16."""
    cases = []
    x = orc.make_inputs(2, 1, 2, 255, 40, seed=1062, primal_scale=2.0, tangent_scale=0.3, dtype=torch.bfloat16)
    cases.append((x, torch.bfloat16, 1e-2))
    x = orc.make_inputs(1, 1, 1, 5, 80, seed=1029, primal_scale=2.0, tangent_scale=0.3, dtype=torch.float16)
    cases.append((x, torch.float16, 0.3))
    x = orc.make_inputs(1, 2, 3, 133, 80, seed=5, primal_scale=1.0, tangent_scale=0.3, dtype=torch.bfloat16)
    for i in range(3):
        x["k"][:, :, 7 + 40 * i, :] = (x["q"][:, :, i, :].float() * 1.5).to(torch.bfloat16)
    cases.append((x, torch.bfloat16, 0.3))
    for x, dtype, unrepaired_floor in cases:
        args = [x[n] for n in orc.TENSOR_ORDER]
        ref = orc.attention_jvp_autograd(*args)
        err = {}
        for label, kw in (("exact", dict(sums_from_outputs=False)), ("delta", dict()), ("repaired", dict(repaired=True))):
            m = orc.row_sum_rounding_model(*args, dtype=dtype, **kw)
            err[label] = {n: orc.rel_frobenius(torch.from_numpy(v), ref[n]) for n, v in m.items()}
        assert max(err["delta"].values()) >= unrepaired_floor, err
        for n in ("dq", "dk", "dtq", "dtk"):
            assert err["repaired"][n] <= 2.0 * err["exact"][n] + 2e-4, (n, err)
            assert err["repaired"][n] <= 5e-3, (n, err)
