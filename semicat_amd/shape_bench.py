"""Step time of the attention-JVP forward + backward at any shape:
``python -m semicat_amd.shape_bench --shape B H L D [--keys Lk] [--dtype bf16|fp16|fp32|fp32io|fp32cast|fp32lib] [--steps K]``.

The same measurement as the headline benchmark (planned launches through the C ABI on one stream,
0.3 s of untimed load first, then K timed steps; random q, k, v ~ 0.5 N(0,1), tangents ~ 0.1 N(0,1),
cotangents ~ N(0,1)), for the shapes the headline benchmark does not cover: longer sequences, other
head dimensions, keys and queries of different lengths.  Work model 42*B*H*Lq*Lk*D flop per step.
Prints one JSON line.  A companion measurement, not the headline figure.

``--dtype fp32`` times the library's fp32 correctness mode (fp32 arithmetic on the vector ALUs);
``--dtype fp32io`` and ``fp32cast`` time the two ways of serving a float32 caller with bf16 arithmetic
(the dtype policy of semicat/jvp_utils/functional.py:318-332): the casts folded into the kernels
(float32 tensors handed over as they are, SJVP_FP32_BF16), or torch casts around the 16-bit kernels
(six casts in, two out in the forward; two in, six out in the backward), or (``fp32lib``) the
library's own multi-tensor cast launches around them, which is what ``safe_sdpa_jvp`` does.
"""
from __future__ import annotations

import argparse
import json
import sys
import time

import torch

from . import _lib, kernels


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--shape", type=int, nargs=4, metavar=("B", "H", "L", "D"), default=(128, 12, 256, 64))
    ap.add_argument("--keys", type=int, default=None, help="key/value length (default: L)")
    ap.add_argument("--dtype", choices=("bf16", "fp16", "fp32", "fp32io", "fp32cast", "fp32lib"), default="bf16")
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("shape_bench needs the GPU", file=sys.stderr)
        return 2
    lib = _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    B, H, Lq, D = a.shape
    Lk = a.keys or Lq
    fp32 = a.dtype.startswith("fp32")
    dt = torch.float32 if fp32 else (torch.bfloat16 if a.dtype == "bf16" else torch.float16)
    code = {"fp32io": _lib.SJVP_FP32_BF16, "fp32": _lib.SJVP_FP32, "fp16": _lib.SJVP_FP16}.get(a.dtype, _lib.SJVP_BF16)
    g = torch.Generator(device=dev).manual_seed(0)

    def rnd(L, s):
        return (torch.randn(B, H, L, D, device=dev, generator=g) * s).to(dt)

    q, tq, dO, dTO = rnd(Lq, 0.5), rnd(Lq, 0.1), rnd(Lq, 1.0), rnd(Lq, 1.0)
    k, v, tk, tv = rnd(Lk, 0.5), rnd(Lk, 0.5), rnd(Lk, 0.1), rnd(Lk, 0.1)
    o, to = torch.empty_like(q), torch.empty_like(q)
    Lr = kernels.stat_rows(Lq)
    lse = torch.empty((B, H, Lr), device=dev, dtype=torch.float32)
    mu = torch.empty_like(lse)
    grads = tuple(torch.empty_like(t) for t in (q, k, v, tq, tk, tv))
    nbytes = lib.sjvp_bwd_workspace_bytes(B, H, Lq, Lk, D, code)
    workspace = torch.empty((max(int(nbytes), 1),), device=dev, dtype=torch.uint8)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        if a.dtype == "fp32lib":
            # the route safe_sdpa_jvp takes for float32 callers: the library's multi-tensor cast launches
            # ([B,S,H,D] views in and out) around the 16-bit kernels
            lo = torch.bfloat16
            bshd = lambda t: t.transpose(1, 2)
            cast = lambda ts, dt_: tuple(bshd(y) for y in kernels.rotary_embedding([bshd(t) for t in ts], None, None,
                                                                                   out_dtype=dt_))
            state = {}

            def fwd():
                a16 = cast((q, k, v), lo) + cast((tq, tk, tv), lo)
                o16, to16, _, _, _ = kernels.attention_jvp_forward(*a16, lse=lse, mu=mu, with_li=False)
                state["saved"] = (a16, o16, to16)
                state["out"] = cast((o16, to16), torch.float32)

            def bwd():
                a16, o16, to16 = state["saved"]
                d16 = cast((dO, dTO), lo)
                g16 = kernels.attention_jvp_backward(*a16, o16, to16, lse, mu, dO=d16[0], dTO=d16[1],
                                                     workspace=workspace)
                state["grads"] = cast(g16[:3], torch.float32) + cast(g16[3:], torch.float32)
        elif a.dtype == "fp32cast":
            lo = torch.bfloat16
            ins16 = [torch.empty_like(t, dtype=lo) for t in (q, k, v, tq, tk, tv)]
            o16, to16, dO16, dTO16 = (torch.empty_like(q, dtype=lo) for _ in range(4))
            grads16 = tuple(torch.empty_like(t, dtype=lo) for t in grads)
            fwd16, _ = kernels.plan_forward(*ins16, o=o16, to=to16, lse=lse, mu=mu, with_li=False)
            bwd16, _ = kernels.plan_backward(*ins16, o16, to16, lse, mu, dO=dO16, dTO=dTO16, grads=grads16,
                                             workspace=workspace)

            def fwd():
                for dst, src in zip(ins16, (q, k, v, tq, tk, tv)):
                    dst.copy_(src)
                fwd16()
                o.copy_(o16)
                to.copy_(to16)

            def bwd():
                dO16.copy_(dO)
                dTO16.copy_(dTO)
                bwd16()
                for dst, src in zip(grads, grads16):
                    dst.copy_(src)
        else:
            arith = {"arithmetic": "bf16"} if a.dtype == "fp32io" else {}
            fwd, _ = kernels.plan_forward(q, k, v, tq, tk, tv, o=o, to=to, lse=lse, mu=mu, with_li=False, **arith)
            bwd, _ = kernels.plan_backward(q, k, v, tq, tk, tv, o, to, lse, mu, dO=dO, dTO=dTO, grads=grads,
                                           workspace=workspace, **arith)
        t_ramp = time.perf_counter() + 0.3  # the clocks settle only under sustained load
        while time.perf_counter() < t_ramp:
            for _ in range(5):
                fwd()
                bwd()
            stream.synchronize()
        for _ in range(a.warmup):
            fwd()
            bwd()
        stream.synchronize()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            fwd()
            bwd()
        stream.synchronize()
        step_ms = (time.perf_counter() - t0) / a.steps * 1e3
        n_ev = min(a.steps, 100)
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n_ev)]
        for e in evs:
            e[0].record(stream)
            fwd()
            e[1].record(stream)
            bwd()
            e[2].record(stream)
        stream.synchronize()
        fwd_ms = sum(e[0].elapsed_time(e[1]) for e in evs) / n_ev
        bwd_ms = sum(e[1].elapsed_time(e[2]) for e in evs) / n_ev
    unit = float(B) * H * Lq * Lk * D
    print(json.dumps({
        "workload": f"attention JVP fwd+bwd, B={B} H={H} Lq={Lq} Lk={Lk} D={D}, "
                    + {"fp32": "fp32 tensors and fp32 arithmetic on the vector ALUs (the correctness mode)",
                       "fp32io": "fp32 tensors, casts folded into the kernels, bf16 arithmetic",
                       "fp32lib": "fp32 tensors, the library's cast launches around the bf16 kernels",
                       "fp32cast": "fp32 tensors, torch casts around the bf16 kernels"}.get(
                           a.dtype, f"{a.dtype} in / fp32 acc") + ", both cotangents",
        "ms_per_step": step_ms, "TFLOPs": 42.0 * unit / (step_ms * 1e-3) / 1e12,
        "fwd_ms": fwd_ms, "fwd_TFLOPs": 12.0 * unit / (fwd_ms * 1e-3) / 1e12,
        "bwd_ms": bwd_ms, "bwd_TFLOPs": 30.0 * unit / (bwd_ms * 1e-3) / 1e12,
        "flop_model": "42*B*H*Lq*Lk*D (forward 12, backward 30)", "steps": a.steps,
        "device": torch.cuda.get_device_name(0), "data": "synthetic",
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())
