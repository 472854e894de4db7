#!/usr/bin/env python3
"""Benchmark of the fused attention-JVP forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--graph] [--no-cpu-baseline] [--no-cold] [--no-hardware] [--no-autograd] [--calib-copy]

A step is one pass of the hot path over one batch: the fused forward (O, TO, lse, mu) followed by
the backward for cotangents on both O and TO (six gradients), on the LM1B-shaped configuration
B=64, H=12, L=128, D=64, bf16 inputs / fp32 accumulation, q,k,v ~ N(0,1)*0.5, tangents ~ N(0,1)*0.1,
cotangents ~ N(0,1), seed 0, inputs resident in HBM.  Throughput uses the work model
42*B*H*L^2*D flop per step (forward 6 + backward 15 tile contractions).  The GPU is first kept busy
for 0.3 s (untimed) so that its clocks have settled, then W warmup steps run, then exactly K steps are
timed.  Prints ONE JSON line.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

METRIC = "JVP-attn fwd+bwd TFLOP/s, % bf16 MFMA peak (B=64,H=12,L=128,D=64)"
B, H, L, D = 64, 12, 128, 64
PRIMAL_SCALE, TANGENT_SCALE, SEED = 0.5, 0.1, 0
PEAK_BF16_TFLOPS = 2500.0   # MI355X dense bf16 MFMA
PEAK_HBM_GBPS = 8000.0      # MI355X HBM3E
NAMES = ("q", "k", "v", "tq", "tk", "tv", "dO", "dTO")
# HBM bytes per launch come from rocprofv3 --pmc runs of this script (FETCH_SIZE, WRITE_SIZE per
# dispatch, scaled by what the same counters read on the copy kernel of --calib-copy); the summary of
# those runs keeps them as "traffic: <kernel> fetch <units> x <KiB per unit> write <units> x <KiB per
# unit> commit <hash>" lines, which is where roofline.traffic is read from.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "kernels_config2_bf16.md")


def measured_traffic(kernel: str):
    """(HBM bytes per launch, source) for a kernel from the committed profiler summary, or (None, None)."""
    try:
        with open(TRAFFIC_FILE) as f:
            for line in f:
                w = line.split()
                if len(w) >= 12 and w[0] == "traffic:" and w[1] == kernel:
                    fetch, fetch_kib, write, write_kib = float(w[3]), float(w[5]), float(w[7]), float(w[9])
                    src = f"profiles/{os.path.basename(TRAFFIC_FILE)} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE at commit {w[11]})"
                    return (fetch * fetch_kib + write * write_kib) * 1024.0, src
    except OSError:
        pass
    return None, None


def cpu_model() -> str:
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def step_flops(b=B, h=H, l=L, d=D) -> float:
    return 42.0 * b * h * l * l * d


def make_inputs(device, b=B):
    """q,k,v,tq,tk,tv,dO,dTO from one CPU generator in this order (fp32 N(0,1), scaled, cast)."""
    g = torch.Generator().manual_seed(SEED)
    out = {}
    for n in NAMES:
        x = torch.randn(b, H, L, D, generator=g, dtype=torch.float32)
        if n in ("q", "k", "v"):
            x *= PRIMAL_SCALE
        elif n in ("tq", "tk", "tv"):
            x *= TANGENT_SCALE
        out[n] = x.to(torch.bfloat16).to(device)
    return out


def _time_cpu(run, seconds: float, max_runs: int = 50):
    run()
    run()
    times = []
    t_end = time.perf_counter() + seconds
    while len(times) < 5 or (time.perf_counter() < t_end and len(times) < max_runs):
        t0 = time.perf_counter()
        run()
        times.append(time.perf_counter() - t0)
    times.sort()
    return times[len(times) // 2], len(times)


def cpu_baseline(seconds: float = 10.0):
    """The reference's CPU math path (torch.func.jvp over eager softmax(QK^T s)V, then autograd for the
    six gradients; oracle.attention_jvp_autograd in fp32) on all host threads torch uses, 2 warm-ups and
    the median of at least 5 runs each: on a bounded sample of the metric's workload (the first 8 of the
    64 batches of config 2, bf16 inputs up-cast to fp32), and on config 1 (B=2, H=4, L=256, D=64, fp32
    N(0,1) inputs, seed 0) in full."""
    from oracle import attn_jvp_oracle as orc
    sample_b = 8
    x = make_inputs("cpu", b=sample_b)
    args = [x[n] for n in NAMES]
    med, n_runs = _time_cpu(lambda: orc.attention_jvp_autograd(*args, dtype=torch.float32), seconds)
    x1 = orc.make_inputs(2, 4, 256, 256, 64, seed=0, dtype=torch.float32)
    args1 = [x1[n] for n in orc.TENSOR_ORDER]
    med1, n1 = _time_cpu(lambda: orc.attention_jvp_autograd(*args1, dtype=torch.float32), seconds / 2)
    return {
        "value": step_flops(b=sample_b) / med / 1e12,
        "unit": "TFLOP/s",
        "cores": torch.get_num_threads(),
        "cpu_model": cpu_model(),
        "kind": "port",
        "sample": f"B={sample_b} of 64 (H=12,L=128,D=64), fp32 eager torch.func.jvp + autograd.grad, "
                  f"median of {n_runs} runs, {med * 1e3:.1f} ms each",
        "config1": {"value": step_flops(2, 4, 256, 64) / med1 / 1e12, "unit": "TFLOP/s",
                    "sample": f"config 1 in full (B=2,H=4,L=256,D=64, fp32, seed 0), median of {n1} runs, "
                              f"{med1 * 1e3:.1f} ms each"},
    }


def autograd_step(x, steps: int = 200):
    """The step as a training loop pays it: torch.func.jvp(sdpa_jvp) and reverse mode through both
    outputs (one forward launch, one backward launch with both cotangents, plus PyTorch's autograd
    machinery on the host).  Wall clock per step over `steps` steps."""
    from semicat_amd import sdpa_jvp
    leaves = [x[n].detach().requires_grad_(True) for n in NAMES[:6]]

    def step():
        y, ty = torch.func.jvp(sdpa_jvp, tuple(leaves[:3]), tuple(leaves[3:]))
        return torch.autograd.grad([y, ty], leaves, [x["dO"], x["dTO"]])

    for _ in range(20):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps * 1e3


def measure_hardware(dev):
    """What this GPU delivers on two plain library workloads, next to the published peaks the
    roofline is priced against: a 1 GiB device-to-device copy (bytes read + written per second) and
    an 8192^3 bf16 GEMM through torch.matmul."""
    props = torch.cuda.get_device_properties(dev)
    src = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    for _ in range(2):
        dst.copy_(src)
    e0.record()
    for _ in range(5):
        dst.copy_(src)
    e1.record()
    e1.synchronize()
    copy_gbps = 5 * 2 * src.numel() / (e0.elapsed_time(e1) * 1e-3) / 1e9
    del src, dst
    n = 8192
    a_ = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    b_ = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
    for _ in range(2):
        a_ @ b_
    e0.record()
    for _ in range(5):
        a_ @ b_
    e1.record()
    e1.synchronize()
    gemm_tflops = 5 * 2.0 * n ** 3 / (e0.elapsed_time(e1) * 1e-3) / 1e12
    return {"compute_units": props.multi_processor_count, "hbm_GiB": props.total_memory / 2 ** 30,
            "copy_GBps": copy_gbps, "bf16_gemm_TFLOPs": gemm_tflops}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--graph", action="store_true",
                    help="replay a HIP graph of one step instead of launching through the C ABI every step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-cold", action="store_true", help="skip the cold-cache timing over rotating buffer sets")
    ap.add_argument("--no-hardware", action="store_true", help="skip the copy / GEMM measurement of the box")
    ap.add_argument("--no-autograd", action="store_true",
                    help="skip timing the step through torch.func.jvp + autograd")
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a 256 MiB device copy (reference point for rocprofv3 --pmc byte counters)")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py: this build targets one GPU; run with --gpus 1 (no multi-GPU path exists: "
              "every (batch, head) pair is an independent problem and shards without communication)",
              file=sys.stderr)
        return 2
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X (torch.cuda.is_available() is False)", file=sys.stderr)
        return 2

    from semicat_amd import _lib, kernels
    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    x = make_inputs(dev)
    q, k, v, tq, tk, tv, dO, dTO = (x[n] for n in NAMES)
    Lr = kernels.stat_rows(L)
    o, to = torch.empty_like(q), torch.empty_like(q)
    lse = torch.empty((B, H, Lr), device=dev, dtype=torch.float32)
    mu = torch.empty_like(lse)
    grads = tuple(torch.empty_like(q) for _ in range(6))

    nbytes = _lib.load().sjvp_bwd_workspace_bytes(B, H, L, L, D, _lib.SJVP_BF16)
    workspace = torch.empty((nbytes,), device=dev, dtype=torch.uint8)

    stream = torch.cuda.Stream()  # default priority; graph capture needs a non-default stream
    graph = None
    with torch.cuda.stream(stream):
        # Planned launches: arguments validated and converted once, each call is one trip through the
        # C ABI (sjvp_fwd, then sjvp_bwd) on this stream.
        fwd, _ = kernels.plan_forward(q, k, v, tq, tk, tv, o=o, to=to, lse=lse, mu=mu, with_li=False)
        bwd, _ = kernels.plan_backward(q, k, v, tq, tk, tv, o, to, lse, mu, dO=dO, dTO=dTO, grads=grads,
                                       workspace=workspace)

        def step():
            fwd()
            bwd()

        # Bring the GPU out of its idle power state before anything is timed: a step lasts tens of
        # microseconds, and the clocks take some hundred milliseconds of load to settle (with 20 warmup
        # steps the same kernels measure 10 % slower than in steady state).
        t_ramp = time.perf_counter() + 0.3
        while time.perf_counter() < t_ramp:
            for _ in range(50):
                step()
            stream.synchronize()
        if a.graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                step()
        run = graph.replay if graph is not None else step

        for _ in range(a.warmup):
            run()
        stream.synchronize()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(a.steps):
            run()
        stream.synchronize()
        torch.cuda.synchronize()
        wall = time.perf_counter() - t0

        # Per-kernel durations: the same steps once more, now with HIP events on the launch stream
        # around every launch (forward and backward alternate exactly as in the timed region, so
        # each kernel meets the caches in the state the other one left them in).
        n_ev = min(a.steps, 200)
        evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(n_ev)]
        for _ in range(3):
            step()
        for e in evs:
            e[0].record(stream)
            fwd()
            e[1].record(stream)
            bwd()
            e[2].record(stream)
        stream.synchronize()
        fwd_each = sorted(e[0].elapsed_time(e[1]) for e in evs)
        bwd_each = sorted(e[1].elapsed_time(e[2]) for e in evs)
        step_each = sorted(e[0].elapsed_time(e[2]) for e in evs)
        fwd_raw_ms = sum(fwd_each) / n_ev
        bwd_raw_ms = sum(bwd_each) / n_ev
        # An event between two kernels keeps them a few microseconds apart, which the plain steps of
        # the timed region do not pay: the instrumented step is that much longer than the timed one.
        # Each kernel's interval holds one such gap; it is taken out in equal parts so that the two
        # durations add up to the step as it was timed.
        gap_ms = max(0.0, (fwd_raw_ms + bwd_raw_ms) - wall / a.steps * 1e3) / 2
        fwd_ms, bwd_ms = fwd_raw_ms - gap_ms, bwd_raw_ms - gap_ms

        # Cold caches: the same step over six independent sets of buffers (1.2 GB in all, several
        # times the 256 MB Infinity Cache) used in rotation, so that no launch finds its operands
        # in a cache; reported beside the headline figure, which re-uses one set as a training
        # step does between a layer's forward and backward.
        cold_ms = None
        if not a.no_cold:
            sets = []
            for _ in range(6):
                y = {n: torch.empty_like(x[n]).copy_(x[n]) for n in NAMES}
                o2, to2 = torch.empty_like(q), torch.empty_like(q)
                lse2, mu2 = torch.empty_like(lse), torch.empty_like(lse)
                g2 = tuple(torch.empty_like(q) for _ in range(6))
                f2, _ = kernels.plan_forward(*(y[n] for n in NAMES[:6]), o=o2, to=to2, lse=lse2, mu=mu2,
                                             with_li=False)
                b2, _ = kernels.plan_backward(*(y[n] for n in NAMES[:6]), o2, to2, lse2, mu2, dO=y["dO"],
                                              dTO=y["dTO"], grads=g2, workspace=workspace)
                sets.append((f2, b2, y, o2, to2, lse2, mu2, g2))
            n_cold = 60
            for i in range(12):
                sets[i % 6][0]()
                sets[i % 6][1]()
            stream.synchronize()
            t0 = time.perf_counter()
            for i in range(n_cold):
                sets[i % 6][0]()
                sets[i % 6][1]()
            stream.synchronize()
            cold_ms = (time.perf_counter() - t0) / n_cold * 1e3
            del sets

        if a.calib_copy:
            # a plain copy of known size, for scaling the FETCH_SIZE / WRITE_SIZE hardware counters
            src = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
            dst = torch.empty_like(src)
            for _ in range(3):
                dst.copy_(src)
            stream.synchronize()

    # the same step through torch.func.jvp + autograd (host-side machinery included)
    autograd_ms = None if a.no_autograd else autograd_step(x)
    hardware = None if a.no_hardware else measure_hardware(dev)
    ms_per_step = wall / a.steps * 1e3
    step_ai = step_flops() / (B * H * (24.0 * L * D * 2 + 16.0 * L))
    tflops = step_flops() / (ms_per_step * 1e-3) / 1e12

    # Algorithmic work per (batch, head), e = 2 bytes.  Forward: 6 tile contractions (12 L^2 D flop);
    # it reads q, k, v and the three tangents and writes O, TO, lse, mu.  Backward: 15 contractions
    # (30 L^2 D flop) in one launch; it reads those six, O, TO, dO, dTO, lse, mu and writes the six
    # gradients: every tensor crosses HBM once.
    BH = B * H
    work = {
        "fwd16_kernel": {"ms": fwd_ms, "flops": 12.0 * BH * L * L * D, "bytes": BH * (8.0 * L * D * 2 + 8.0 * L)},
        "bwd_fused16_kernel": {"ms": bwd_ms, "flops": 30.0 * BH * L * L * D,
                               "bytes": BH * (16.0 * L * D * 2 + 8.0 * L)},
    }
    for w in work.values():
        w["GBps"] = w["bytes"] / (w["ms"] * 1e-3) / 1e9
        w["TFLOPs"] = w["flops"] / (w["ms"] * 1e-3) / 1e12
    dom = max(work, key=lambda n: work[n]["ms"])
    dk = work[dom]
    ridge = PEAK_BF16_TFLOPS * 1e12 / (PEAK_HBM_GBPS * 1e9)
    if dk["flops"] / dk["bytes"] < ridge:
        roofline = {"bound": "hbm", "achieved": dk["GBps"], "peak": PEAK_HBM_GBPS, "unit": "GB/s",
                    "frac": dk["GBps"] / PEAK_HBM_GBPS}
    else:
        roofline = {"bound": "mfma", "achieved": dk["TFLOPs"], "peak": PEAK_BF16_TFLOPS, "unit": "TFLOP/s",
                    "frac": dk["TFLOPs"] / PEAK_BF16_TFLOPS}
    # HBM bytes per launch of the dominant kernel from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of
    # this script (scaled by the same counters on the --calib-copy kernel).
    roofline["traffic"], roofline["traffic_source"] = measured_traffic(dom)
    roofline["kernel"] = dom
    roofline["ms"] = dk["ms"]
    roofline["algorithmic_bytes"] = dk["bytes"]
    roofline["algorithmic_flops"] = dk["flops"]
    roofline["flop_per_byte"] = dk["flops"] / dk["bytes"]

    out = {
        "metric": METRIC,
        "value": tflops,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "config 2: LM1B-shaped DiT attention JVP fwd+bwd, B=64 H=12 L=128 D=64, "
                               "bf16 in / fp32 acc, non-causal, both cotangents",
                   "launch": "one sjvp_fwd + one sjvp_bwd call per step" if graph is None
                             else "hip-graph replay of one fwd+bwd step",
                   "flop_model": "42*B*H*L^2*D"},
        "pct_mfma_peak": 100.0 * tflops / PEAK_BF16_TFLOPS,
        # the step's own roof: min(MFMA peak, flop per algorithmic byte of the step x HBM peak)
        "pct_of_min_mfma_hbm_roof": 100.0 * tflops / min(PEAK_BF16_TFLOPS, step_ai * PEAK_HBM_GBPS / 1e3),
        "step_flop_per_byte": step_ai,
        "autograd_step_ms": autograd_ms,
        "fwd_ms": fwd_ms,
        "bwd_ms": bwd_ms,
        "event_intervals_ms": {"fwd": fwd_raw_ms, "bwd": bwd_raw_ms, "gap_removed_per_kernel": gap_ms,
                               # median and minimum over the instrumented steps (event gaps included)
                               "fwd_median": fwd_each[n_ev // 2], "fwd_min": fwd_each[0],
                               "bwd_median": bwd_each[n_ev // 2], "bwd_min": bwd_each[0],
                               "step_median": step_each[n_ev // 2], "step_min": step_each[0]},
        # the forward by the count of the reference's own harness (10*B*H*L^2*D, ryu_triton.py:1000-1003,
        # which under-counts its six contractions), for comparison with figures quoted that way
        "fwd_TFLOPs_by_reference_count": 10.0 * BH * L * L * D / (fwd_ms * 1e-3) / 1e12,
        "cold_ms_per_step": cold_ms,
        "cold_tflops": None if cold_ms is None else step_flops() / (cold_ms * 1e-3) / 1e12,
        "kernels": {n: {"ms": w["ms"], "GBps": w["GBps"], "TFLOPs": w["TFLOPs"]} for n, w in work.items()},
        "roofline": roofline,
        "device": torch.cuda.get_device_name(0),
        "hardware": hardware,
    }
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())
