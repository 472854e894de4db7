"""Step time of the DiT training step that surrounds the attention-JVP op:
``python -m semicat_amd.dit_bench [--batch 64] [--sd-prop 0.25] [--steps 5] [--warmup 2]``.

Workload: the reference's LM1B DiT (12 blocks, width 768, 12 heads of 64, conditioning width 128,
sequence 128, vocabulary 30522; configs/model/text8_dit_lg.yaml:8-15,
configs/experiment/lm1b_dit.yaml:15-23), random initial weights, uniformly random token ids,
Gaussian prior, bf16 autocast, AdamW.  One step = both losses of ``train_step.model_step``, backward,
optimizer step.  ``--sd-prop`` is the share of the batch that takes the self-distillation loss
(forward-mode AD through the network, reference default 0.25; 1.0 makes every attention call have the
shape B=64, H=12, L=128, D=64).

Prints one JSON line with the step time and the time spent inside the attention kernels (HIP events
around every launch of the op on the current stream).  This is a companion measurement of the code
around the op, not the headline benchmark.
"""
from __future__ import annotations

import argparse
import json
import sys

import torch

from . import kernels, train_step
from .dit import DIT


class _KernelTimer:
    """Wraps the launchers of :mod:`semicat_amd.kernels` with HIP event pairs."""

    NAMES = ("attention_jvp_forward", "attention_jvp_backward", "attention_forward")

    def __init__(self):
        self.pairs: list[tuple[str, torch.cuda.Event, torch.cuda.Event]] = []
        self._orig = {}

    def __enter__(self):
        for name in self.NAMES:
            orig = getattr(kernels, name)
            self._orig[name] = orig

            def timed(*a, _orig=orig, _name=name, **kw):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                out = _orig(*a, **kw)
                e1.record()
                self.pairs.append((_name, e0, e1))
                return out

            setattr(kernels, name, timed)
        return self

    def __exit__(self, *exc):
        for name, orig in self._orig.items():
            setattr(kernels, name, orig)

    def totals_ms(self) -> dict[str, float]:
        torch.cuda.synchronize()
        out: dict[str, float] = {}
        for name, e0, e1 in self.pairs:
            out[name] = out.get(name, 0.0) + e0.elapsed_time(e1)
        return out


def rope_only(args, dev) -> int:
    """q and k of one block rotated out of the fused bf16 qkv projection into contiguous bf16
    tensors: one launch reads and writes 2 * B*S*H*D 16-bit elements each way."""
    from .dit import Rotary
    B, S, H, D = args.batch, args.length, 12, 64
    cos, sin = Rotary(S, D).to(dev).half_tables()
    qkv = torch.randn(B, S, 3, H, D, device=dev).to(torch.bfloat16)
    xs = (qkv[:, :, 0], qkv[:, :, 1])
    import time
    t_ramp = time.perf_counter() + 0.3  # the GPU leaves its idle power state only under sustained load
    while time.perf_counter() < t_ramp:
        for _ in range(20):
            kernels.rotary_embedding(xs, cos, sin)
        torch.cuda.synchronize()
    n = 200
    # launches are enqueued faster than they run only for large batches; time the stream as a whole
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(n):
        kernels.rotary_embedding(xs, cos, sin)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) / n * 1e3
    nbytes = 2 * 2 * B * S * H * D * 2 + 2 * S * (D // 2) * 4
    print(json.dumps({"workload": f"rotary embedding of q and k, B={B} S={S} H={H} D={D}, bf16 -> bf16",
                      "us_per_launch": us, "algorithmic_bytes": nbytes, "GBps": nbytes / us / 1e3,
                      "frac_of_8TBps": nbytes / us / 1e3 / 8000.0}))
    return 0


def graph_step(args, net, opt, x1) -> int:
    """The whole step captured once and replayed: forward-mode AD through the network, the attention
    and rotary launches of the library, the backward and AdamW all become nodes of one HIP graph (the
    library allocates nothing, records no memset and never synchronises, so its launches can be
    captured).  The replay time is what the kernels of a step take without the host issuing them one
    by one.  The random draws of a step come from the default generator, which graph capture
    advances per replay."""
    def step():
        opt.zero_grad(set_to_none=False)
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            vf, sd = train_step.model_step(net, x1, (args.length, args.vocab), sd_prop=args.sd_prop)
        loss = vf if sd is None else (sd if int(args.sd_prop * args.batch) == args.batch else vf + sd)
        loss.backward()
        opt.step()
        return vf.detach(), None if sd is None else sd.detach()

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(max(3, args.warmup)):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        vf, sd = step()
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(args.steps):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    print(json.dumps({
        "workload": f"LM1B DiT step: {args.blocks} blocks, width 768, 12x64 heads, seq {args.length}, "
                    f"vocab {args.vocab}, batch {args.batch}, sd_prop {args.sd_prop}, bf16 autocast, AdamW",
        "launch": "HIP graph replay of one whole step",
        "ms_per_step": e0.elapsed_time(e1) / args.steps,
        "plain_attention": args.plain_attention, "rotary": args.rotary,
        "vfm_loss": float(vf), "sd_loss": None if sd is None else float(sd),
        "max_memory_GB": torch.cuda.max_memory_allocated() / 2**30,
        "data": "synthetic (uniform token ids, random weights)",
    }))
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--sd-prop", type=float, default=0.25)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--vocab", type=int, default=30522)
    ap.add_argument("--length", type=int, default=128)
    ap.add_argument("--blocks", type=int, default=12)
    ap.add_argument("--plain-attention", choices=("hip", "torch"), default="hip")
    ap.add_argument("--rotary", choices=("hip", "torch"), default="hip")
    ap.add_argument("--graph", action="store_true",
                    help="capture one whole step (losses, backward, AdamW) in a HIP graph and time its replays")
    ap.add_argument("--rope-only", action="store_true",
                    help="time only the rotary kernel on q and k of one block (batch x length x 12 heads of 64)")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("dit_bench needs the GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.manual_seed(0)
    if args.rope_only:
        return rope_only(args, dev)
    net = DIT(vocab_size=args.vocab, hidden_size=768, cond_dim=128, n_blocks=args.blocks, n_heads=12,
              dropout=0.1, length=args.length, plain_attention=args.plain_attention,
              rotary=args.rotary).to(dev)
    # the reference zero-initialises the output projection and the modulations (duo.py:124-125,188-194),
    # which makes the first step's attention gradients vanish; start from a generic point instead
    for p in net.parameters():
        if not p.any():
            torch.nn.init.normal_(p, std=0.02)
    opt = torch.optim.AdamW(net.parameters(), lr=1e-4, weight_decay=0.0, capturable=args.graph)
    gen = torch.Generator(device=dev).manual_seed(0)
    x1 = torch.randint(0, args.vocab, (args.batch, args.length), device=dev, generator=gen)

    if args.graph:
        return graph_step(args, net, opt, x1)

    def step():
        opt.zero_grad(set_to_none=True)
        with torch.autocast(device_type="cuda", dtype=torch.bfloat16):
            vf, sd = train_step.model_step(net, x1, (args.length, args.vocab), sd_prop=args.sd_prop,
                                           generator=gen)
        # with sd_prop = 1 the cross-entropy share of the batch is empty and its mean is NaN
        # (semicat.py:186-187 behaves the same): leave it out of the loss then
        loss = vf if sd is None else (sd if int(args.sd_prop * args.batch) == args.batch else vf + sd)
        loss.backward()
        opt.step()
        return vf.detach(), None if sd is None else sd.detach()

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    with _KernelTimer() as timer:
        e0.record()
        for _ in range(args.steps):
            vf, sd = step()
        e1.record()
        torch.cuda.synchronize()
        step_ms = e0.elapsed_time(e1) / args.steps
        per_kernel = {k: v / args.steps for k, v in timer.totals_ms().items()}
    attn_ms = sum(per_kernel.values())
    print(json.dumps({
        "workload": f"LM1B DiT step: {args.blocks} blocks, width 768, 12x64 heads, seq {args.length}, "
                    f"vocab {args.vocab}, batch {args.batch}, sd_prop {args.sd_prop}, bf16 autocast, AdamW",
        "ms_per_step": step_ms,
        "attention_ms_per_step": attn_ms,
        "attention_share": attn_ms / step_ms,
        "attention_launch_ms": per_kernel,
        "plain_attention": args.plain_attention,
        "rotary": args.rotary,
        "vfm_loss": float(vf), "sd_loss": None if sd is None else float(sd),
        "max_memory_GB": torch.cuda.max_memory_allocated() / 2**30,
        "data": "synthetic (uniform token ids, random weights)",
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())
