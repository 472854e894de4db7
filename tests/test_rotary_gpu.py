"""GPU tests of the rotary kernel (sjvp_rope through semicat_amd.kernels.rotary_embedding and the
autograd function in semicat_amd.rotary) against the oracle's complex-arithmetic rotation in fp64
(oracle/rotary_oracle.py) and, for the two AD modes, against autograd through the PyTorch formula
(semicat_amd.dit.rotate_half_embedding, pinned on the CPU against the same oracle).  Bars: one rounding of the output dtype (bf16 2^-8, fp16 2^-11 relative to the row
scale) and 2e-6 for fp32 output."""
import pytest
import torch

from oracle import rotary_oracle as ro
from semicat_amd.dit import Rotary, rotate_half_embedding

pytestmark = pytest.mark.gpu

TOL = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2e-6}


@pytest.fixture(scope="module")
def K():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import semicat_amd.kernels as kernels
    from semicat_amd import _lib
    _lib.load()
    return kernels


def tables(S, rot, device="cuda"):
    r = Rotary(S, rot).to(device)
    return r.half_tables()  # strided views of the [1,S,3,1,rot] buffers (row stride 3*rot)


def oracle_rotation(x, cos, sin, inverse=False):
    """fp64 rotation of a [B,S,H,D] tensor by the angles the fp32 tables encode."""
    theta = torch.atan2(sin.double(), cos.double()).cpu().numpy()
    return torch.from_numpy(ro.rotate(x.double().cpu().numpy(), theta, inverse=inverse))


def check(y, ref, dtype):
    err = (y.double().cpu() - ref.cpu()).abs().max().item()
    assert err <= TOL[dtype] * max(1.0, ref.abs().max().item()), (err, dtype)


@pytest.mark.parametrize("in_dtype,out_dtype", [
    (torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16), (torch.float32, torch.bfloat16),
    (torch.float32, torch.float32), (torch.bfloat16, torch.float32), (torch.float32, torch.float16)])
@pytest.mark.parametrize("B,S,H,D,rot", [(2, 128, 12, 64, 64), (1, 50, 3, 128, 64), (2, 33, 2, 20, 20),
                                         (1, 7, 1, 48, 32)])
def test_rotation_matches_the_fp64_formula(K, in_dtype, out_dtype, B, S, H, D, rot):
    torch.manual_seed(0)
    cos, sin = tables(S, rot)
    # q and k as slices of a fused projection, as in duo.py:137-138
    qkv = torch.randn(B, S, 3, H, D, device="cuda").to(in_dtype)
    q, k = qkv[:, :, 0], qkv[:, :, 1]
    yq, yk = K.rotary_embedding((q, k), cos, sin, out_dtype=out_dtype)
    assert yq.is_contiguous() and yq.dtype == out_dtype and yq.shape == (B, S, H, D)
    for x, y in ((q, yq), (k, yk)):
        check(y, oracle_rotation(x, cos, sin), out_dtype)
    # the inverse rotation undoes it (up to the roundings of the two passes)
    back, = K.rotary_embedding((yq,), cos, sin, out_dtype=torch.float32, inverse=True)
    assert (back.double() - q.double()).abs().max().item() <= 3 * TOL[out_dtype] * max(1.0, q.abs().max().item())


def test_one_to_four_tensors_and_argument_checks(K):
    torch.manual_seed(1)
    cos, sin = tables(16, 32)
    xs = [torch.randn(1, 16, 2, 32, device="cuda", dtype=torch.bfloat16) for _ in range(4)]
    for n in (1, 3, 4):
        ys = K.rotary_embedding(xs[:n], cos, sin)
        for x, y in zip(xs, ys):
            check(y, oracle_rotation(x, cos, sin), torch.bfloat16)
    with pytest.raises(ValueError):
        K.rotary_embedding(xs + xs[:1], cos, sin)
    with pytest.raises(AssertionError):
        K.rotary_embedding((xs[0], xs[1][:, :8]), cos, sin)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        K.rotary_embedding((xs[0].cpu(),), cos.cpu(), sin.cpu())
    empty = K.rotary_embedding((xs[0][:0],), cos, sin)[0]
    assert empty.shape == (0, 16, 2, 32)


def test_both_ad_modes_through_the_kernel(K):
    """torch.func.jvp over the kernel, then reverse mode through primal and tangent outputs, against
    autograd through the PyTorch formula."""
    from semicat_amd.rotary import apply_rotary
    torch.manual_seed(2)
    B, S, H, D = 2, 40, 3, 64
    cos, sin = tables(S, D)
    mk = lambda: torch.randn(B, S, H, D, device="cuda", dtype=torch.float32)
    q, k, tq, tk, wq, wk, wtq = mk(), mk(), mk(), mk(), mk(), mk(), mk()

    def run(fn):
        a, b, ta, tb = (t.clone().requires_grad_(True) for t in (q, k, tq, tk))
        (ya, yb), (tya, tyb) = torch.func.jvp(fn, (a, b), (ta, tb))
        ((ya * wq).sum() + (yb * wk).sum() + (tya * wtq).sum() + (tyb ** 2).sum()).backward()
        return [t.detach() for t in (ya, yb, tya, tyb)] + [a.grad, b.grad, ta.grad, tb.grad]

    got = run(lambda a, b: apply_rotary((a, b), cos, sin))
    ref = run(lambda a, b: (rotate_half_embedding(a, cos, sin), rotate_half_embedding(b, cos, sin)))
    for g, r in zip(got, ref):
        assert g.shape == r.shape and torch.allclose(g, r, rtol=1e-5, atol=1e-5)
    # a tensor without tangent, a single tensor, and a 16-bit pipeline
    ya, tya = torch.func.jvp(lambda a: apply_rotary(a, cos, sin), (q,), (tq,))
    assert torch.allclose(tya, rotate_half_embedding(tq, cos, sin), rtol=1e-5, atol=1e-5)
    xb = q.to(torch.bfloat16).requires_grad_(True)
    yb = apply_rotary(xb, cos, sin)
    assert yb.dtype == torch.bfloat16
    yb.float().pow(2).sum().backward()
    assert xb.grad.dtype == torch.bfloat16
    # R is orthogonal: the gradient of |R x|^2 is 2 x
    assert (xb.grad.float() - 2 * xb.detach().float()).abs().max().item() <= 0.05 * xb.abs().max().item()


# ------------------------------------------------------------------------------------------------
# The rotation folded into the attention launches (sjvp_fwd_rotary / sjvp_bwd_rotary).

GRADS = ("dq", "dk", "dv", "dtq", "dtk", "dtv")


def _rot_bhld(x, cos, sin, inverse=False):
    """oracle rotation of a [B,H,L,D] tensor (the oracle speaks [B,S,H,D])."""
    return oracle_rotation(x.transpose(1, 2), cos, sin, inverse=inverse).transpose(1, 2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("mode", ["both", "dO", "dTO"])
@pytest.mark.parametrize("B,H,Lq,Lk", [(2, 3, 128, 128), (1, 2, 100, 77), (1, 2, 200, 128), (2, 1, 31, 17)])
def test_rotation_folded_into_the_attention_launches(K, dtype, mode, B, H, Lq, Lk):
    """q, k and their tangents handed over UNROTATED as strided slices of a fused projection, with the
    tables: outputs equal attention on the oracle-rotated inputs, and the gradients are those with
    respect to the unrotated tensors (the oracle's gradients of the rotated ones, rotated back)."""
    from oracle import attn_jvp_oracle as orc
    D = 64
    x = orc.make_inputs(B, H, Lq, Lk, D, seed=51, tangent_scale=0.3, dtype=dtype)
    cos, sin = tables(max(Lq, Lk), D)
    rot = {n: (_rot_bhld(x[n], cos, sin) if n in ("q", "k", "tq", "tk") else x[n].double()) for n in x}
    cot = {}
    if mode != "dTO":
        cot["dO"] = x["dO"]
    if mode != "dO":
        cot["dTO"] = x["dTO"]
    ref = orc.attention_jvp_autograd(*[rot[n] for n in orc.TENSOR_ORDER[:6]], **cot)
    for n in ("dq", "dk", "dtq", "dtk"):
        ref[n] = _rot_bhld(ref[n], cos, sin, inverse=True)
    # k-side and q-side tensors as [B,H,L,D] views of [B,L,3,H,D] buffers (the fused projection's layout)
    def fused_view(names, L):
        buf = torch.zeros(B, L, 3, H, D, device="cuda", dtype=dtype)
        for i, n in enumerate(names):
            buf[:, :, i] = x[n].cuda().transpose(1, 2)
        return [buf[:, :, i].transpose(1, 2) for i in range(len(names))]
    q, tq = fused_view(("q", "tq"), Lq)
    k, v = fused_view(("k", "v"), Lk)
    tk, tv = fused_view(("tk", "tv"), Lk)
    assert K.rotary_fusable(q, k, cos, [v, tq, tk, tv])
    o, to, lse, mu, _ = K.attention_jvp_forward(q, k, v, tq, tk, tv, rope=(cos, sin))
    dO, dTO = x["dO"].cuda(), x["dTO"].cuda()
    if mode == "dO":
        g = K.attention_jvp_backward(q, k, v, None, None, None, o, None, lse, None, dO=dO, rope=(cos, sin))
    else:
        g = K.attention_jvp_backward(q, k, v, tq, tk, tv, o, to, lse, mu, dO=dO if mode == "both" else None,
                                     dTO=dTO, rope=(cos, sin))
    torch.cuda.synchronize()
    res = {"O": o, "TO": to, **{n: t for n, t in zip(GRADS, g) if t is not None}}
    errs = {}
    for n, t in res.items():
        assert torch.isfinite(t.float()).all(), n
        errs[n] = orc.rel_frobenius(t.cpu(), ref[n])
    print(f"[folded rotary {dtype} {mode} {(B, H, Lq, Lk)}] " + " ".join(f"{n}={e:.2e}" for n, e in errs.items()),
          flush=True)
    assert all(e <= 1e-2 for e in errs.values()), errs
    # the primal-only forward with the same folding
    o2, lse2 = K.attention_forward(q, k, v, rope=(cos, sin))
    assert orc.rel_frobenius(o2.cpu(), ref["O"]) <= 1e-2
    assert torch.allclose(lse2[..., :Lq], lse[..., :Lq], rtol=1e-5, atol=1e-5)
    # and the two-launch way (rotary kernel, then the plain attention kernels) agrees
    qr, tqr = (t.transpose(1, 2) for t in K.rotary_embedding((q.transpose(1, 2), tq.transpose(1, 2)), cos, sin))
    kr, tkr = (t.transpose(1, 2) for t in K.rotary_embedding((k.transpose(1, 2), tk.transpose(1, 2)), cos, sin))
    o3, to3, _, _, _ = K.attention_jvp_forward(qr, kr, v, tqr, tkr, tv)
    assert orc.rel_frobenius(o3.cpu(), o.cpu()) <= 2e-3 and orc.rel_frobenius(to3.cpu(), to.cpu()) <= 4e-3


def test_shapes_the_folded_rotation_does_not_serve_are_refused(K):
    from semicat_amd import _lib
    cos, sin = tables(256, 64)
    z = lambda L, D=64: torch.zeros(1, 1, L, D, device="cuda", dtype=torch.bfloat16)
    for q, k in ((z(64), z(256)), (z(64, 32), z(64, 32))):
        assert not K.rotary_fusable(q, k, cos)
        with pytest.raises(_lib.SjvpError, match="rotary"):
            K.attention_jvp_forward(q, k, k, q, k, k, rope=(cos, sin))
    assert not K.rotary_fusable(z(64).float(), z(64).float(), cos)
    # tables the launchers would reject are refused here too, so that callers fall back instead of raising
    q = z(64)
    assert K.rotary_fusable(q, q, cos, sin=sin)
    assert not K.rotary_fusable(q, q, cos[:32], sin=sin[:32])                 # fewer rows than positions
    assert not K.rotary_fusable(q, q, cos, sin=sin.double())                   # sin of another dtype
    assert not K.rotary_fusable(q, q, cos, sin=sin.cpu())                      # sin on another device
    assert not K.rotary_fusable(q, q, cos, sin=torch.zeros(256, 64, device="cuda")[:, ::2])  # strided columns
    assert not K.rotary_fusable(q, q, cos.reshape(-1)[1:1 + 255 * 32].view(255, 32))  # misaligned table
    assert not K.rotary_fusable(q, q, cos[None])                               # not two-dimensional


def test_network_block_issues_no_rotary_launch_at_sequence_128():
    """The DiT at the training configuration's attention shape (12 heads of 64, sequence 128): with the
    rotation folded into the attention launches no rotary kernel runs, in either AD mode."""
    from torch.profiler import ProfilerActivity, profile
    from semicat_amd import train_step as ts
    from semicat_amd.dit import DIT
    torch.manual_seed(0)
    net = DIT(vocab_size=64, hidden_size=768, cond_dim=32, n_blocks=2, n_heads=12, dropout=0.0, length=128).cuda()
    for p in net.parameters():
        if not p.any():
            torch.nn.init.normal_(p, std=0.05)
    x1 = torch.randint(0, 64, (4, 128), device="cuda")
    x0 = torch.randn(4, 128, 64, device="cuda")
    with profile(activities=[ProfilerActivity.CUDA]) as prof:
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            loss = ts.lag_self_distillation_loss(net, x0, x1) + ts.vfm_loss(net, x0, x1)
        loss.backward()
        torch.cuda.synchronize()
    names = [e.key for e in prof.key_averages() if e.device_type == torch.autograd.DeviceType.CUDA]
    assert any("fwd16_kernel" in n for n in names) and any("bwd_fused" in n for n in names), names
    assert not any("rope_kernel" in n for n in names), [n for n in names if "rope" in n]
