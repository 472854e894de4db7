#!/usr/bin/env python3
"""Writes tests/golden/attn_jvp_fp64.npz: expected outputs of the attention-JVP path for small seeded
inputs, evaluated in fp64 by the oracle's autograd math path (oracle/attn_jvp_oracle.py, which is
pinned independently in tests/test_oracle.py).  The reference repository holds no golden vectors for
this path and is not imported here; the shapes, seed and value scales are those of its own forward
test (semicat/jvp_utils/ryu_triton.py:501-524) plus one ragged case.

Inputs are not stored: tests regenerate them with oracle.make_inputs(seed, ...) and compare.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import attn_jvp_oracle as orc  # noqa: E402

CASES = {
    # name: (B, H, Lq, Lk, D, seed, tangent_scale, input dtype)
    "ref_1x1x8x16": (1, 1, 8, 8, 16, 42, 0.1, torch.float16),
    "ref_2x2x16x32": (2, 2, 16, 16, 32, 42, 0.1, torch.float16),
    "ref_1x4x32x32": (1, 4, 32, 32, 32, 42, 0.1, torch.float16),
    "ragged_1x2x37x53x16": (1, 2, 37, 53, 16, 7, 1.0, torch.bfloat16),
}
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "attn_jvp_fp64.npz")


def main():
    blob = {}
    for name, (B, H, Lq, Lk, D, seed, ts, dt) in CASES.items():
        x = orc.make_inputs(B, H, Lq, Lk, D, seed=seed, tangent_scale=ts, dtype=dt)
        res = orc.attention_jvp_autograd(*[x[n] for n in orc.TENSOR_ORDER])
        cf = orc.attention_jvp_closed_form(*[x[n] for n in orc.TENSOR_ORDER[:6]])
        for k in ("O", "TO", "dq", "dk", "dv", "dtq", "dtk", "dtv"):
            blob[f"{name}/{k}"] = res[k].numpy()
        blob[f"{name}/lse"] = cf["lse"]
        blob[f"{name}/mu"] = cf["mu"]
    np.savez_compressed(OUT, **blob)
    print(f"wrote {OUT}: {len(blob)} arrays, {os.path.getsize(OUT) / 1024:.0f} KiB")


if __name__ == "__main__":
    main()
