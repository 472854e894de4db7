"""CPU oracle for the rotary position embedding in front of the attention-JVP op.  TEST
INFRASTRUCTURE ONLY: imported by ``tests/`` alone; the product (``semicat_amd``) never routes
through it.

What it restates (reference = olsdavis/semicat): ``Rotary`` and
``split_and_apply_rotary_pos_emb`` (semicat/net/duo.py:24-55), which rotate q and k with
``flash_attn.layers.rotary.apply_rotary_emb_torch`` of the un-vendored dependency flash_attn
(environment.yaml pins 2.8.3; absent from the reference tree and from this image).  That routine's
published non-interleaved algorithm: with ``ro = 2 * cos.shape[-1]``, ``x1 = x[..., :ro/2]`` and
``x2 = x[..., ro/2:ro]``, the result is ``[x1 cos - x2 sin | x2 cos + x1 sin | x[..., ro:]]``; the
angle at position ``l`` and pair ``i`` is ``l * base^(-2 i / dim)`` (duo.py:27-31).

It is evaluated here through complex arithmetic in numpy fp64 - ``(x1 + j x2) * exp(j theta)`` - so
that a sign or pairing mistake in an implementation written with real cos / sin products does not
cancel against the same mistake here.

Pinning status: the mathematics is pinned in tests/test_dit_step.py (norm preservation, the inverse
rotation, scores depending on the position difference only, agreement with the real-arithmetic
formula).  Parity with the reference's own rotary routine is UNPINNED: the reference holds no test
or fixture for it, and the routine lives in a dependency that cannot be imported here.
"""
from __future__ import annotations

import numpy as np


def rotary_angles(seq_len: int, dim: int, base: float = 10_000.0) -> np.ndarray:
    """``theta[l, i] = l * base^(-2i/dim)`` for ``i < dim/2`` (duo.py:27-30)."""
    inv_freq = base ** (-np.arange(0, dim, 2, dtype=np.float64) / dim)
    return np.arange(seq_len, dtype=np.float64)[:, None] * inv_freq[None, :]


def rotate(x: np.ndarray, theta: np.ndarray, inverse: bool = False) -> np.ndarray:
    """``x`` ``[B,S,H,D]`` rotated by ``theta`` ``[S, ro/2]``, pairing column ``i`` with ``i + ro/2``;
    columns from ``ro`` on are unchanged."""
    x = np.asarray(x, dtype=np.float64)
    half = theta.shape[-1]
    z = x[..., :half] + 1j * x[..., half:2 * half]
    z = z * np.exp((-1j if inverse else 1j) * theta)[None, :x.shape[1], None, :]
    return np.concatenate((z.real, z.imag, x[..., 2 * half:]), axis=-1)
