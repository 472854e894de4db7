"""The DiT and the training-step losses around the attention-JVP op (semicat_amd/dit.py,
semicat_amd/train_step.py).

CPU tests: the rotary restatement against an independent complex-number formulation, the parameter
names a reference checkpoint would carry (duo.py:101-202, 299-343), the interpolation and loss
formulas against direct evaluation, and the wiring of the whole self-distillation step through the op
(kernel launchers replaced by the eager stand-ins of tests/eager_backend.py).
GPU tests: the same step with the HIP kernels against the same network with eager math attention.

The reference holds no test or fixture for the network or the step, and its rotary comes from the
un-vendored flash_attn 2.8.3: parity of these layers with the reference is unpinned; what is pinned
here is their mathematics and the behaviour of the op inside them."""
import math

import pytest
import torch
import torch.nn.functional as F

from semicat_amd import train_step as ts
from semicat_amd.dit import DIT, Rotary, math_attention, rotate_half_embedding

from . import eager_backend


def make_net(vocab=48, hidden=64, heads=2, blocks=2, length=16, cond=16, seed=0, **kw):
    torch.manual_seed(seed)
    kw.setdefault("rotary", "torch")  # the CPU tests; the GPU tests ask for the HIP rotary kernel
    net = DIT(vocab_size=vocab, hidden_size=hidden, cond_dim=cond, n_blocks=blocks, n_heads=heads,
              dropout=0.0, length=length, **kw)
    # the zero-initialised modulation and output layers would make the output independent of attention
    for p in net.parameters():
        if not p.any():
            torch.nn.init.normal_(p, std=0.05)
    return net


def test_rotary_is_a_complex_rotation_and_relative():
    """The real-arithmetic rotation of the product against the oracle's complex formulation, and the
    properties that fix the oracle itself: it preserves norms, its inverse undoes it, the identity
    slice for v, a partial rotary width, and scores that depend on the position difference only."""
    import numpy as np
    from oracle import rotary_oracle as ro
    torch.manual_seed(0)
    S, D = 12, 16
    rot = Rotary(S, D)
    cos, sin = rot.half_tables()
    assert cos.shape == (S, D // 2) and rot.cos_cached.shape == (1, S, 3, 1, D)
    assert torch.all(rot.cos_cached[:, :, 2] == 1) and torch.all(rot.sin_cached[:, :, 2] == 0)
    theta = ro.rotary_angles(S, D)
    assert np.allclose(np.cos(theta), cos.double().numpy(), atol=1e-6)  # the buffers are fp32
    x = torch.randn(2, S, 3, D, dtype=torch.float64)
    c64, s64 = torch.from_numpy(np.cos(theta)), torch.from_numpy(np.sin(theta))
    out = rotate_half_embedding(x, c64, s64)
    ref = ro.rotate(x.numpy(), theta)
    assert np.allclose(out.numpy(), ref, atol=1e-12)
    assert np.allclose(np.linalg.norm(ref, axis=-1), np.linalg.norm(x.numpy(), axis=-1), atol=1e-12)
    assert np.allclose(ro.rotate(ref, theta, inverse=True), x.numpy(), atol=1e-12)
    assert np.allclose(ref[:, 0], x.numpy()[:, 0], atol=1e-12)  # position 0 is the identity
    # partial rotary width: the columns beyond it pass through
    part = rotate_half_embedding(x, c64[:, :4], s64[:, :4])
    assert np.allclose(part.numpy(), ro.rotate(x.numpy(), theta[:, :4]), atol=1e-12)
    assert torch.equal(part[..., 8:], x[..., 8:])
    # scores depend on the position difference only
    q, k = np.random.default_rng(0).standard_normal((2, D))
    qa = ro.rotate(np.broadcast_to(q, (1, S, 1, D)), theta)[0, :, 0]
    ka = ro.rotate(np.broadcast_to(k, (1, S, 1, D)), theta)[0, :, 0]
    scores = qa @ ka.T
    assert np.isclose(scores[3, 1], scores[9, 7], atol=1e-9) and np.isclose(scores[0, 5], scores[6, 11], atol=1e-9)


def test_state_dict_names_match_a_reference_checkpoint():
    net = make_net(vocab=30, hidden=32, heads=2, blocks=1, length=8, cond=8)
    names = {n: tuple(t.shape) for n, t in net.state_dict().items()}
    expected = {
        "vocab_embed.seq.weight": (32, 30), "vocab_embed.seq.bias": (32,),
        "s_map.mlp.0.weight": (8, 256), "s_map.mlp.2.weight": (8, 8), "s_map.freqs": (128,),
        "t_map.mlp.0.bias": (8,), "t_map.mlp.2.bias": (8,), "t_map.freqs": (128,),
        "rotary_emb.cos_cached": (1, 8, 3, 1, 16), "rotary_emb.sin_cached": (1, 8, 3, 1, 16),
        "blocks.0.norm1.weight": (32,), "blocks.0.attn_qkv.weight": (96, 32), "blocks.0.attn_out.weight": (32, 32),
        "blocks.0.norm2.bias": (32,), "blocks.0.mlp.0.weight": (128, 32), "blocks.0.mlp.2.bias": (32,),
        "blocks.0.adaLN_modulation.weight": (192, 8), "blocks.0.adaLN_modulation.bias": (192,),
        "output_layer.norm_final.weight": (32,), "output_layer.linear.weight": (30, 32),
        "output_layer.adaLN_modulation.weight": (64, 8),
    }
    for n, shape in expected.items():
        assert names.get(n) == shape, n
    assert "blocks.0.attn_qkv.bias" not in names and "blocks.0.attn_out.bias" not in names
    fresh = DIT(30, 32, 8, 1, 2, 0.1, 8)
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        fresh(torch.zeros(1, 8, 30), torch.zeros(1), torch.ones(1))  # rotary="hip" needs the GPU
    assert not fresh.output_layer.linear.weight.any() and not fresh.blocks[0].adaLN_modulation.weight.any()


def test_interpolate_and_losses_against_direct_evaluation():
    torch.manual_seed(1)
    B, S, V = 3, 16, 48
    x1 = torch.randint(0, V, (B, S))
    x0 = torch.randn(B, S, V)
    t = torch.rand(B)
    xt = ts.interpolate(x0, x1, t.view(B, 1, 1))
    assert torch.allclose(xt, (1 - t.view(B, 1, 1)) * x0 + t.view(B, 1, 1) * F.one_hot(x1, V).float(), atol=1e-6)
    net = make_net(attention_override=math_attention)
    loss = ts.vfm_loss(net, x0, x1, t=t)
    logits = net(xt, t, t)
    direct = -(torch.log_softmax(logits, -1).gather(-1, x1[..., None])).mean()
    assert torch.allclose(loss, direct, atol=1e-5)
    # the reference's formulation (class axis second), also with label smoothing
    assert torch.allclose(loss, F.cross_entropy(logits.transpose(-1, 1), x1), atol=1e-6)
    assert torch.allclose(ts.vfm_loss(net, x0, x1, label_smoothing=0.1, t=t),
                          F.cross_entropy(logits.transpose(-1, 1), x1, label_smoothing=0.1), atol=1e-6)
    # the time derivative inside the self-distillation loss against a central difference in fp64
    net64 = make_net(attention_override=math_attention).double()
    s = torch.rand(B, dtype=torch.float64) * t.double()
    xs = ts.interpolate(x0.double(), x1, s.view(B, 1, 1))
    f = lambda end: ts.flow_map(net64, xs, s, end)
    _, dv = torch.func.jvp(f, (t.double(),), (torch.ones(B, dtype=torch.float64),))
    eps = 1e-5
    fd = (f(t.double() + eps) - f(t.double() - eps)) / (2 * eps)
    assert torch.allclose(dv, fd, atol=1e-6, rtol=1e-5)
    loss = ts.lag_self_distillation_loss(net64, x0.double(), x1, t=t.double(), s=s)
    xst = f(t.double()).detach()
    target = net64(xst, t.double(), t.double()).softmax(-1)
    direct = (((1 - t.double().view(B, 1, 1)) * fd - target + xst) ** 2).sum(-1).mean()
    assert torch.allclose(loss, direct, rtol=1e-5)
    assert ts.sample_prior((2, 4, 5), "cpu", "discunif").sum(-1).eq(1).all()
    vf, sd = ts.model_step(net, x1, (S, V), sd_prop=0.0)
    assert sd is None and torch.isfinite(vf)


def _step_losses_and_grads(net, x0, x1, t, s):
    net.zero_grad(set_to_none=True)
    split = x1.shape[0] // 2
    sd = ts.lag_self_distillation_loss(net, x0[:split], x1[:split], t=t[:split], s=s[:split])
    vf = ts.vfm_loss(net, x0[split:], x1[split:], t=t[split:])
    (vf + 10.0 * sd).backward()
    grads = {n: p.grad.detach().float().clone() for n, p in net.named_parameters()}
    return vf.item(), sd.item(), grads


def _compare_steps(net, device, autocast, loss_tol, grad_tol):
    torch.manual_seed(2)
    B, S, V = 4, net.blocks[0].seq_len, net.vocab_size
    x1 = torch.randint(0, V, (B, S), device=device)
    x0 = torch.randn(B, S, V, device=device)
    t = torch.rand(B, device=device)
    s = torch.rand(B, device=device) * t
    results = []
    for override, rotary in ((None, net.rotary), (math_attention, "torch")):
        net.attention_override, net.rotary = override, rotary
        with torch.autocast(device_type=device, dtype=torch.bfloat16, enabled=autocast):
            results.append(_step_losses_and_grads(net, x0, x1, t, s))
    (vf_a, sd_a, g_a), (vf_b, sd_b, g_b) = results
    assert math.isfinite(vf_a) and math.isfinite(sd_a)
    assert abs(vf_a - vf_b) <= loss_tol * abs(vf_b), (vf_a, vf_b)
    assert abs(sd_a - sd_b) <= loss_tol * abs(sd_b), (sd_a, sd_b)
    for n in g_a:
        if "attn" in n or "mlp" in n or "vocab_embed" in n:
            err = (g_a[n] - g_b[n]).norm() / g_b[n].norm()
            assert err <= grad_tol, (n, err.item())


def test_self_distillation_step_through_the_op_cpu(monkeypatch):
    """torch.func.jvp over the network with the op inside, then reverse mode through the tangent:
    same losses and gradients as with eager math attention (the op rounds its inputs to bf16)."""
    eager_backend.install(monkeypatch)
    net = make_net()
    _compare_steps(net, "cpu", autocast=False, loss_tol=2e-2, grad_tol=8e-2)


def test_step_with_the_rotation_folded_into_the_op_cpu(monkeypatch):
    """The network hands q, k unrotated to safe_sdpa_jvp_rotary; with the launchers replaced by eager
    stand-ins that apply the rotation themselves (and the inverse rotation to the gradients), losses
    and gradients equal those of eager math attention behind the PyTorch rotary."""
    from semicat_amd import kernels
    eager_backend.install(monkeypatch)
    monkeypatch.setattr(kernels, "rotary_fusable", lambda *a, **kw: True)
    net = make_net(rotary="hip")
    _compare_steps(net, "cpu", autocast=False, loss_tol=2e-2, grad_tol=8e-2)


@pytest.mark.gpu
def test_self_distillation_step_through_the_op_gpu():
    """As above with the HIP kernels, under bf16 autocast as in the reference's training configuration
    (configs/experiment/lm1b_dit.yaml:15), heads of 64 and sequence length 128."""
    from semicat_amd import _lib
    _lib.load()
    net = make_net(vocab=96, hidden=128, heads=2, blocks=2, length=128, cond=32, rotary="hip").cuda()
    _compare_steps(net, "cuda", autocast=True, loss_tol=3e-2, grad_tol=1e-1)


@pytest.mark.gpu
@pytest.mark.parametrize("sd_prop", [0.25, 1.0])
def test_full_size_step_gpu(sd_prop):
    """The training configuration at its real size (configs/model/text8_dit_lg.yaml:8-15,
    configs/experiment/lm1b_dit.yaml:15-23): 12 blocks, d_model 768, 12 heads of 64, cond_dim 128,
    sequence 128, vocabulary 30522, batch 64, bf16 autocast, random token ids.  The first
    int(sd_prop * 64) samples take the self-distillation loss through the HIP attention-JVP and
    rotary kernels, the others the cross-entropy loss (semicat.py:186-191; the reference default is
    sd_prop = 0.25, and sd_prop = 1 makes every attention call the benchmark's shape).  Losses finite
    and equal to the same network with eager math attention and the PyTorch rotary."""
    from semicat_amd import _lib
    _lib.load()
    B, S, V = 64, 128, 30522
    print(f"[full-size step] sd_prop={sd_prop}", flush=True)
    net = make_net(vocab=V, hidden=768, heads=12, blocks=12, length=S, cond=128, rotary="hip").cuda()
    torch.manual_seed(5)
    x1 = torch.randint(0, V, (B, S), device="cuda")
    x0 = torch.randn(B, S, V, device="cuda")
    t = torch.rand(B, device="cuda")
    s = torch.rand(B, device="cuda") * t
    split = int(sd_prop * B)
    watched = ("blocks.0.attn_qkv.weight", "blocks.11.attn_qkv.weight", "blocks.5.mlp.0.weight",
               "vocab_embed.seq.weight")
    results = []
    for override, rotary in ((None, "hip"), (math_attention, "torch")):
        net.attention_override, net.rotary = override, rotary
        net.zero_grad(set_to_none=True)
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            sd = ts.lag_self_distillation_loss(net, x0[:split], x1[:split], t=t[:split], s=s[:split])
            vf = ts.vfm_loss(net, x0[split:], x1[split:], t=t[split:]) if split < B else None
        (sd if vf is None else vf + sd).backward()
        params = dict(net.named_parameters())
        results.append((sd.item(), None if vf is None else vf.item(),
                        {n: params[n].grad.detach().float().clone() for n in watched}))
        torch.cuda.synchronize()
    (sd_a, vf_a, g_a), (sd_b, vf_b, g_b) = results
    print(f"[full-size step] sd {sd_a:.6g} vs {sd_b:.6g}; vfm {vf_a} vs {vf_b}", flush=True)
    assert math.isfinite(sd_a) and abs(sd_a - sd_b) <= 3e-2 * abs(sd_b), (sd_a, sd_b)
    if vf_a is not None:
        assert math.isfinite(vf_a) and abs(vf_a - vf_b) <= 3e-2 * abs(vf_b), (vf_a, vf_b)
    for n in watched:
        assert torch.isfinite(g_a[n]).all(), n
        err = ((g_a[n] - g_b[n]).norm() / g_b[n].norm()).item()
        print(f"[full-size step] grad {n}: rel err {err:.3e}", flush=True)
        assert err <= 1e-1, (n, err)


@pytest.mark.gpu
def test_plain_attention_modes_agree_gpu():
    from semicat_amd import _lib
    _lib.load()
    net = make_net(vocab=96, hidden=128, heads=2, blocks=2, length=128, cond=32).cuda()
    torch.manual_seed(3)
    x = torch.randn(4, 128, 96, device="cuda")
    t = torch.rand(4, device="cuda")
    outs = {}
    for mode in ("hip", "torch"):
        net.plain_attention = mode
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            outs[mode] = net(x, 0.5 * t, t).float()
    err = (outs["hip"] - outs["torch"]).norm() / outs["torch"].norm()
    assert err < 2e-2, err.item()


@pytest.mark.gpu
def test_network_under_torch_compile_gpu():
    """The reference compiles the network (semicat.py:340-345) and keeps the op opaque to dynamo
    (functional.py:272): with the network wrapped by torch.compile, the cross-entropy step (compiled
    graph with a break at the op) and the self-distillation step (forward-mode AD over the wrapped
    network) give the results of the unwrapped network.  The aot_eager backend exercises dynamo and
    AOTAutograd without generating device code."""
    from semicat_amd import _lib
    _lib.load()
    net = make_net(vocab=96, hidden=128, heads=2, blocks=2, length=128, cond=32, rotary="hip").cuda()
    torch.manual_seed(4)
    x1 = torch.randint(0, 96, (4, 128), device="cuda")
    x0 = torch.randn(4, 128, 96, device="cuda")
    t = torch.rand(4, device="cuda")
    s = torch.rand(4, device="cuda") * t

    def run(n):
        net.zero_grad(set_to_none=True)
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            vf = ts.vfm_loss(n, x0, x1, t=t)
            sd = ts.lag_self_distillation_loss(n, x0, x1, t=t, s=s)
        (vf + sd).backward()
        return vf.item(), sd.item(), net.blocks[0].attn_qkv.weight.grad.clone()

    vf0, sd0, g0 = run(net)
    torch._dynamo.reset()
    vf1, sd1, g1 = run(torch.compile(net, backend="aot_eager"))
    assert abs(vf1 - vf0) <= 1e-5 * abs(vf0) and abs(sd1 - sd0) <= 1e-5 * abs(sd0)
    assert (g1 - g0).norm() <= 1e-5 * g0.norm()


def test_compile_network_refuses_inductor_on_a_gpu_and_passes_other_backends_through():
    """The helper that wraps the network as the reference does: "aot_eager" (and anything on the CPU) goes
    to torch.compile, inductor for a network on a GPU raises before anything is compiled."""
    from semicat_amd.train_step import compile_network
    net = torch.nn.Linear(4, 4)
    compiled = compile_network(net, backend="aot_eager")
    x = torch.randn(2, 4)
    assert torch.allclose(compiled(x), net(x))

    class OnGpu(torch.nn.Module):  # stands for a network whose parameters live on a GPU
        def parameters(self, recurse=True):
            class P:
                is_cuda = True
            return iter([P()])

    with pytest.raises(RuntimeError, match="inductor"):
        compile_network(OnGpu(), backend="inductor")


@pytest.mark.gpu
@pytest.mark.skip(reason="torch.compile(net, backend='inductor') on an MI355X box ended in a segmentation fault of "
                         "the Python process while inductor compiled the PyTorch layers around the op (torch "
                         "2.10.0+rocm7.0, triton 3.6.0); no cause has been shown, so the case stays off the GPU. "
                         "On the CPU inductor compiles the network and matches eager, and triton 3.6.0 "
                         "cross-compiles a kernel for gfx950 without a GPU.")
def test_network_under_inductor_gpu():
    from semicat_amd.train_step import compile_network  # noqa: F401
    raise AssertionError("not run: see the skip reason")
