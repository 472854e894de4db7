"""The committed fp64 fixtures (tests/golden/attn_jvp_fp64.npz, written by tests/golden/make_fixtures.py)
against every CPU implementation of the oracle, and - on the GPU - against the HIP kernels."""
import os

import numpy as np
import pytest
import torch

from oracle import attn_jvp_oracle as orc
from oracle import c_ref
from tests.golden.make_fixtures import CASES, OUT

OUTS = ("O", "TO", "dq", "dk", "dv", "dtq", "dtk", "dtv")


@pytest.fixture(scope="module")
def golden():
    assert os.path.exists(OUT), "run tests/golden/make_fixtures.py"
    return np.load(OUT, allow_pickle=False)


def _inputs(name):
    B, H, Lq, Lk, D, seed, ts, dt = CASES[name]
    return orc.make_inputs(B, H, Lq, Lk, D, seed=seed, tangent_scale=ts, dtype=dt)


@pytest.mark.parametrize("name", list(CASES))
def test_cpu_implementations_reproduce_the_fixtures(golden, name):
    x = _inputs(name)
    a = [x[n] for n in orc.TENSOR_ORDER]
    for impl in (orc.attention_jvp_closed_form, c_ref.attention_jvp_c):
        res = impl(*a)
        for k in OUTS:
            assert orc.rel_frobenius(res[k], golden[f"{name}/{k}"]) < 1e-12, (impl.__name__, k)
    if max(x["q"].shape[2], x["k"].shape[2]) <= 16 and x["q"].shape[0] == 1:
        bf = orc.attention_jvp_bruteforce(*[t[0, 0] for t in a])
        for k in OUTS:
            assert orc.rel_frobenius(bf[k], golden[f"{name}/{k}"][0, 0]) < 1e-12, k


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(CASES))
def test_hip_kernels_against_the_fixtures(golden, name):
    import semicat_amd.kernels as K
    x = _inputs(name)
    d = {n: t.cuda() for n, t in x.items()}
    o, to, lse, mu, _ = K.attention_jvp_forward(d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"])
    g = K.attention_jvp_backward(d["q"], d["k"], d["v"], d["tq"], d["tk"], d["tv"], o, to, lse, mu,
                                 dO=d["dO"], dTO=d["dTO"])
    res = dict(zip(OUTS, (o, to) + tuple(g)))
    for k in OUTS:
        err = orc.rel_frobenius(res[k].cpu(), golden[f"{name}/{k}"])
        assert err <= 1e-2, (k, err)  # 16-bit kernels: relative Frobenius <= 1e-2
    Lq = x["q"].shape[2]
    np.testing.assert_allclose(lse[..., :Lq].cpu().numpy(), golden[f"{name}/lse"], rtol=2e-5, atol=2e-5)
