"""CPU tests of the host side: the autograd wiring of sdpa_jvp / safe_sdpa_jvp (with the kernel
launchers replaced by eager stand-ins from tests/eager_backend.py), argument checking, and the C-ABI
library's exported symbols.  No HIP compute call is made here."""
import ctypes
import os
import re

import pytest
import torch

import semicat_amd
from semicat_amd import _lib, build, functional, kernels
from oracle import attn_jvp_oracle as orc

from . import eager_backend

GRADS = ("dq", "dk", "dv", "dtq", "dtk", "dtv")


def _leaf(x, dtype):
    return x.to(dtype).clone().requires_grad_(True)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 3e-2)])
def test_jvp_then_backward_both_cotangents(monkeypatch, dtype, tol):
    """torch.func.jvp(sdpa_jvp) then reverse mode through BOTH outputs reaches all six inputs and
    equals the oracle's autograd path (drop-in contract of functional.py:298-301)."""
    eager_backend.install(monkeypatch)
    x = orc.make_inputs(2, 2, 24, 40, 16, seed=1, dtype=dtype)
    leaves = [_leaf(x[n], dtype) for n in orc.TENSOR_ORDER[:6]]
    y, ty = torch.func.jvp(functional.sdpa_jvp, tuple(leaves[:3]), tuple(leaves[3:]))
    assert y.shape == (2, 2, 24, 16) and y.is_contiguous() and ty.shape == y.shape
    (y.float() * x["dO"].float()).sum().add((ty.float() * x["dTO"].float()).sum()).backward()
    ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
    assert orc.rel_frobenius(y, ref["O"]) < tol and orc.rel_frobenius(ty, ref["TO"]) < tol
    for n, leaf in zip(GRADS, leaves):
        assert leaf.grad is not None, n
        assert orc.rel_frobenius(leaf.grad, ref[n]) < tol, n


@pytest.mark.parametrize("wiring,launches", [("fused", 1), ("reference", 2)])
def test_autograd_wirings_agree_and_differ_in_backward_launches(monkeypatch, wiring, launches):
    """Both wirings of the op give the oracle's gradients; the fused node runs the backward as ONE
    launch with both cotangents, the reference's arrangement (functional.py:52-87, 216-268) as two
    launches with one cotangent each."""
    eager_backend.install(monkeypatch)
    monkeypatch.setattr(functional, "AUTOGRAD_WIRING", wiring)
    calls = []
    real = kernels.attention_jvp_backward

    def spy(*a, dO=None, dTO=None, **kw):
        calls.append((dO is not None, dTO is not None))
        return real(*a, dO=dO, dTO=dTO, **kw)

    monkeypatch.setattr(kernels, "attention_jvp_backward", spy)
    x = orc.make_inputs(2, 2, 24, 40, 16, seed=4)
    leaves = [_leaf(x[n], torch.float32) for n in orc.TENSOR_ORDER[:6]]
    y, ty = torch.func.jvp(functional.sdpa_jvp, tuple(leaves[:3]), tuple(leaves[3:]))
    ((y * x["dO"]).sum() + (ty * x["dTO"]).sum()).backward()
    assert len(calls) == launches
    assert (True, True) in calls if wiring == "fused" else sorted(calls) == [(False, True), (True, False)]
    ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
    for n, leaf in zip(GRADS, leaves):
        assert orc.rel_frobenius(leaf.grad, ref[n]) < 2e-5, n
    # one cotangent only: the other output's branch is skipped (set_materialize_grads(False))
    calls.clear()
    leaves = [_leaf(x[n], torch.float32) for n in orc.TENSOR_ORDER[:6]]
    y, ty = torch.func.jvp(functional.sdpa_jvp, tuple(leaves[:3]), tuple(leaves[3:]))
    (y * x["dO"]).sum().backward()
    assert calls == [(True, False)]
    assert all(leaf.grad is None for leaf in leaves[3:])


@pytest.mark.parametrize("which", ["primal", "tangent"])
def test_single_cotangent(monkeypatch, which):
    """Only one of the two autograd nodes receives a cotangent (set_materialize_grads(False),
    functional.py:237,263-264)."""
    eager_backend.install(monkeypatch)
    x = orc.make_inputs(1, 2, 16, 16, 16, seed=2)
    leaves = [_leaf(x[n], torch.float32) for n in orc.TENSOR_ORDER[:6]]
    y, ty = torch.func.jvp(functional.sdpa_jvp, tuple(leaves[:3]), tuple(leaves[3:]))
    if which == "primal":
        (y * x["dO"]).sum().backward()
        ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER[:6]], dO=x["dO"])
        for leaf in leaves[3:]:
            assert leaf.grad is None
        names = GRADS[:3]
    else:
        (ty * x["dTO"]).sum().backward()
        ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER[:6]], dTO=x["dTO"])
        names = GRADS
    for n, leaf in zip(names, leaves):
        assert orc.rel_frobenius(leaf.grad, ref[n]) < 2e-5, n


def test_plain_forward_and_backward_without_tangents(monkeypatch):
    """Without forward-mode tangents the op is ordinary attention (the reference returns garbage
    here, functional.py:286-287)."""
    eager_backend.install(monkeypatch)
    x = orc.make_inputs(1, 2, 16, 24, 16, seed=3)
    q, k, v = (_leaf(x[n], torch.float32) for n in "qkv")
    y = functional.sdpa_jvp(q, k, v)
    (y * x["dO"]).sum().backward()
    ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER[:6]], dO=x["dO"])
    assert orc.rel_frobenius(y, ref["O"]) < 2e-5
    for n, leaf in zip(GRADS[:3], (q, k, v)):
        assert orc.rel_frobenius(leaf.grad, ref[n]) < 2e-5, n


def test_safe_sdpa_jvp_layout_and_dtype(monkeypatch):
    """[B,S,H,D] in and out; fp32 inputs are computed in bf16 and come back as fp32
    (functional.py:318-332): with FP32_CALLERS = "folded" the casts are folded into the launch (the
    launcher gets the fp32 tensors and arithmetic="bf16"), with the default "torch" the launcher gets
    bf16 tensors; other dtypes are cast with torch.  Inside the op q,k,v are [B,H,S,D] views with strides
    (S*H*D, D, H*D, 1)."""
    seen = {}
    real = eager_backend.attention_jvp_forward

    def spy(q, k, v, *a, **kw):
        seen["strides"] = q.stride()
        seen["dtype"] = q.dtype
        seen["arithmetic"] = kw.get("arithmetic")
        return real(q, k, v, *a, **kw)

    eager_backend.install(monkeypatch)
    monkeypatch.setattr(kernels, "attention_jvp_forward", spy)
    B, S, H, D = 2, 8, 3, 16
    g = torch.Generator().manual_seed(0)
    q, k, v, tq, tk, tv = (torch.randn(B, S, H, D, generator=g) for _ in range(6))
    ref = orc.attention_jvp_autograd(*(t.transpose(1, 2) for t in (q, k, v, tq, tk, tv)))
    assert functional.FP32_CALLERS == "torch"
    for dtype, want, route in ((torch.float32, (torch.float32, "bf16"), "folded"),
                               (torch.float32, (torch.bfloat16, None), "torch"),
                               (torch.float64, (torch.bfloat16, None), "torch")):
        monkeypatch.setattr(functional, "FP32_CALLERS", route)
        y, ty = torch.func.jvp(functional.safe_sdpa_jvp, tuple(t.to(dtype) for t in (q, k, v)),
                               tuple(t.to(dtype) for t in (tq, tk, tv)))
        assert y.shape == (B, S, H, D) and y.dtype == dtype and ty.dtype == dtype
        assert seen["strides"] == (S * H * D, D, H * D, 1)
        assert (seen["dtype"], seen["arithmetic"]) == want
        assert orc.rel_frobenius(y.transpose(1, 2), ref["O"]) < 3e-2
        assert orc.rel_frobenius(ty.transpose(1, 2), ref["TO"]) < 3e-2
    # precise=True keeps fp32 tensors and fp32 arithmetic
    y, ty = torch.func.jvp(lambda a, b, c: functional.safe_sdpa_jvp(a, b, c, precise=True), (q, k, v), (tq, tk, tv))
    assert (seen["dtype"], seen["arithmetic"]) == (torch.float32, None)
    assert orc.rel_frobenius(ty.transpose(1, 2), ref["TO"]) < 2e-5


def test_through_a_module_with_scalar_time_tangent(monkeypatch):
    """The training pattern (semicat.py:153-157): jvp w.r.t. a scalar time through a block that
    modulates the attention input, then backward to the block's weights."""
    eager_backend.install(monkeypatch)
    torch.manual_seed(0)
    lin = torch.nn.Linear(16, 48)
    x = torch.randn(2, 8, 16)

    def net(t):
        h = lin(x * (1 + t))
        q, k, v = h.view(2, 8, 3, 2, 8).permute(2, 0, 1, 3, 4).unbind(0)  # [B,S,H,D] each... D=8 -> pad
        q, k, v = (torch.cat([z, z], -1) for z in (q, k, v))              # D = 16
        return functional.safe_sdpa_jvp(q.contiguous(), k.contiguous(), v.contiguous())

    t = torch.tensor(0.3)
    y, ty = torch.func.jvp(net, (t,), (torch.ones(()),))
    (y.sum() + (ty ** 2).sum()).backward()
    assert lin.weight.grad is not None and torch.isfinite(lin.weight.grad).all()
    assert lin.weight.grad.abs().sum() > 0


def test_seq_major_results_need_no_copy(monkeypatch):
    """safe_sdpa_jvp hands back [B,S,H,D]-contiguous results (primal and tangent, with and without
    forward-mode AD), so flattening the heads as duo.py:155 does is a view; sdpa_jvp keeps the
    reference's [B,H,S,D]-contiguous result (functional.py:224-227)."""
    eager_backend.install(monkeypatch)
    x = orc.make_inputs(2, 3, 12, 12, 16, seed=3, dtype=torch.bfloat16)
    bshd = [x[n].transpose(1, 2).contiguous() for n in orc.TENSOR_ORDER[:6]]
    y, ty = torch.func.jvp(functional.safe_sdpa_jvp, tuple(bshd[:3]), tuple(bshd[3:]))
    plain = functional.safe_sdpa_jvp(*bshd[:3])
    for t in (y, ty, plain):
        assert t.shape == (2, 12, 3, 16) and t.is_contiguous()
        assert t.reshape(2, 12, 48).data_ptr() == t.data_ptr()
    ref = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
    assert orc.rel_frobenius(y.transpose(1, 2), ref["O"]) < 3e-2
    assert orc.rel_frobenius(ty.transpose(1, 2), ref["TO"]) < 3e-2
    assert orc.rel_frobenius(plain.transpose(1, 2), ref["O"]) < 3e-2
    y2, _ = torch.func.jvp(functional.sdpa_jvp, tuple(x[n] for n in orc.TENSOR_ORDER[:3]),
                           tuple(x[n] for n in orc.TENSOR_ORDER[3:6]))
    assert y2.is_contiguous() and y2.shape == (2, 3, 12, 16)


def test_launchers_refuse_cpu_tensors():
    """No CPU fallback: the real launchers raise on non-GPU tensors."""
    q = torch.zeros(1, 1, 8, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.attention_jvp_forward(q, q, q, q, q, q)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.attention_forward(q, q, q)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.attention_jvp_backward(q, q, q, q, q, q, q, q, None, None, dTO=q)


def test_library_exports_every_declared_symbol(repo_root):
    """libsjvp.so loads and exports exactly what include/sjvp.h declares; the functions that need
    no GPU answer."""
    header = open(os.path.join(repo_root, "include", "sjvp.h")).read()
    declared = set(re.findall(r"\b(sjvp_[a-z_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTS)
    if build.is_stale():
        build.build()
    assert build.built_id() == build.source_id()
    lib = ctypes.CDLL(build.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    L = _lib.load()
    assert L.sjvp_version() == int(re.search(r"#define SJVP_VERSION (\d+)", header).group(1))
    # 12 bytes per statistic row (rows rounded up to 128 per head) + one 4-byte flag per 64 rows
    assert L.sjvp_bwd_workspace_bytes(64, 12, 128, 128, 64, 0) == 3 * 64 * 12 * 128 * 4 + 64 * 12 * 2 * 4
    assert L.sjvp_bwd_workspace_bytes(1, 1, 129, 7, 64, 0) == 3 * 256 * 4 + 4 * 4
    for code in range(0, -12, -1):
        assert _lib.strerror(code) and "unknown" not in _lib.strerror(code)
    assert "unknown" in _lib.strerror(-99)


def test_c_abi_argument_errors_are_reported_before_any_launch():
    """Argument validation happens on the host before any HIP call, so it can be exercised
    without a GPU: bad head dims, dtype, shapes, NULLs, missing cotangents, small workspace."""
    L = _lib.load()
    strides = (ctypes.c_int64 * 48)(*([0] * 48))
    one = ctypes.c_void_p(16)  # non-NULL placeholder; never dereferenced on these paths
    f = lambda **kw: L.sjvp_fwd(one, one, one, one, one, one, one, one, one, one, one,
                                kw.get("B", 1), 1, kw.get("Lq", 8), 8, kw.get("D", 64), strides, 0.0,
                                kw.get("dtype", 0), None)
    assert f(D=8) == _lib.SJVP_ERR_HEAD_DIM       # ryu_triton.py:319-322
    assert f(D=256) == _lib.SJVP_ERR_HEAD_DIM     # flash_jvp_backward.py:2318
    assert f(dtype=7) == _lib.SJVP_ERR_DTYPE
    assert f(B=0) == _lib.SJVP_ERR_SHAPE
    assert f(Lq=0) == _lib.SJVP_ERR_SHAPE
    # scale: 0 selects 1/sqrt(D); negative, infinite and NaN are refused
    for bad in (-1.0, float("inf"), float("nan")):
        assert L.sjvp_fwd(one, one, one, one, one, one, one, one, one, one, one, 1, 1, 8, 8, 64, strides,
                          bad, 0, None) == _lib.SJVP_ERR_SCALE
    for bad in (0.0, -0.5, float("inf")):
        with pytest.raises(ValueError):
            kernels._scale_arg(bad)
    assert kernels._scale_arg(None) == 0.0 and kernels._scale_arg(0.125) == 0.125
    assert L.sjvp_fwd(None, one, one, one, one, one, one, one, one, one, one, 1, 1, 8, 8, 64, strides,
                      0.0, 0, None) == _lib.SJVP_ERR_NULL
    # tangent inputs must come all together
    assert L.sjvp_fwd(one, one, one, one, None, one, one, one, one, one, one, 1, 1, 8, 8, 64, strides,
                      0.0, 0, None) == _lib.SJVP_ERR_NULL
    b = lambda dO, dTO, ws, nbytes: L.sjvp_bwd(one, one, one, one, one, one, one, one, dO, dTO, one,
                                              one, one, one, one, one, one, one, ws, nbytes, 1, 1, 8,
                                              8, 64, strides, 0.0, 0, None)
    assert b(None, None, one, 1 << 20) == _lib.SJVP_ERR_COTANGENT
    assert b(one, one, None, 1 << 20) == _lib.SJVP_ERR_WORKSPACE
    assert b(one, one, one, 8) == _lib.SJVP_ERR_WORKSPACE
    # the no-allocation backward refuses what its static scratch cannot hold, before any HIP call
    assert L.sjvp_bwd_noalloc(*([one] * 18), 64, 16, 1025, 128, 64, strides, 0.0, 0, None) == _lib.SJVP_ERR_SCRATCH
    assert L.sjvp_bwd_noalloc(*([one] * 8), None, None, *([one] * 8), 1, 1, 8, 8, 64, strides, 0.0, 0,
                              None) == _lib.SJVP_ERR_COTANGENT
    with pytest.raises(_lib.SjvpError):
        _lib.check(_lib.SJVP_ERR_HEAD_DIM)
    # sjvp_rope
    ptrs = (ctypes.c_void_p * 4)(16, 16, 16, 16)
    rs = (ctypes.c_int64 * 24)(*([0] * 24))
    r = lambda **kw: L.sjvp_rope(kw.get("n", 2), kw.get("x", ptrs), ptrs, rs, kw.get("cos", one), one, 32, 1, 1,
                                 kw.get("L", 8), 64, kw.get("rot", 64), kw.get("i", 0), kw.get("o", 0), 0, None)
    assert r(n=0) == _lib.SJVP_ERR_ROTARY and r(n=5) == _lib.SJVP_ERR_ROTARY
    assert r(rot=63) == _lib.SJVP_ERR_ROTARY and r(rot=66) == _lib.SJVP_ERR_ROTARY and r(rot=-2) == _lib.SJVP_ERR_ROTARY
    assert r(i=0, o=1) == _lib.SJVP_ERR_ROTARY  # bf16 in, fp16 out
    assert r(i=5) == _lib.SJVP_ERR_DTYPE
    assert r(L=0) == _lib.SJVP_ERR_SHAPE
    assert r(cos=None) == _lib.SJVP_ERR_NULL
    assert r(x=(ctypes.c_void_p * 4)(16, None, 16, 16)) == _lib.SJVP_ERR_NULL


def test_companion_benchmarks_refuse_to_run_without_gpu(capsys):
    """The companion benchmarks measure the HIP path only: without a GPU they say so and return 2."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from semicat_amd import dit_bench, shape_bench
    assert shape_bench.main(["--shape", "2", "2", "64", "64"]) == 2
    assert dit_bench.main([]) == 2
    assert "needs the GPU" in capsys.readouterr().err
