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
