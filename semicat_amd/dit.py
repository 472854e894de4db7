"""The DiT that calls the attention-JVP op, as plain PyTorch modules around
:func:`semicat_amd.functional.safe_sdpa_jvp`.

It restates the network of olsdavis/semicat's ``semicat/net/duo.py`` (cited by line below) so that
the op can be exercised where the reference calls it: twelve times per step, from inside
``torch.func.jvp`` over the whole network, under bf16 autocast, with reverse mode through both the
primal and the tangent.  Module and parameter names follow the reference (``vocab_embed.seq``,
``s_map.mlp.{0,2}``, ``blocks.<i>.attn_qkv`` ...), so a reference ``state_dict`` loads unchanged.

Only the arithmetic of attention runs in HIP kernels; every other layer is stock PyTorch.

Rotary embedding: the reference calls ``flash_attn.layers.rotary.apply_rotary_emb_torch`` (duo.py:52-53;
flash_attn 2.8.3, not vendored).  :func:`rotate_half_embedding` restates that routine's published
non-interleaved form: with ``x = [x1 | x2]`` split at half the head dimension,
``out = [x1 cos - x2 sin | x2 cos + x1 sin]``.  The rotation is linear in ``x``, so forward-mode AD
carries tangents through it with the same formula.
"""
from __future__ import annotations

import math
from typing import Callable, Optional

import torch
import torch.nn.functional as F
from torch import Tensor, nn

from .functional import safe_sdpa_jvp, safe_sdpa_jvp_rotary
from .rotary import apply_rotary


def math_attention(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
    """softmax(q k^T / sqrt(D)) v on ``[B,S,H,D]`` with differentiable torch ops (works under both AD
    modes); the comparison path of the tests, never used by default."""
    qh, kh, vh = (t.transpose(1, 2) for t in (q, k, v))
    scores = torch.matmul(qh, kh.transpose(-1, -2)) / math.sqrt(q.shape[-1])
    return torch.matmul(torch.softmax(scores, dim=-1), vh).transpose(1, 2)


def rotate_half_embedding(x: Tensor, cos: Tensor, sin: Tensor) -> Tensor:
    """Rotary position embedding of ``x`` ``[B,S,H,D]`` with ``cos``/``sin`` ``[S,D/2]``, pairing
    element ``i`` with element ``i + D/2`` (duo.py:49-53)."""
    half = cos.shape[-1]
    c = cos[None, :, None, :]
    s = sin[None, :, None, :]
    x1, x2, rest = x[..., :half], x[..., half:2 * half], x[..., 2 * half:]
    return torch.cat((x1 * c - x2 * s, x2 * c + x1 * s, rest), dim=-1)


class Rotary(nn.Module):
    """Cached cos/sin tables in the reference's buffer layout ``[1,S,3,1,D]`` (duo.py:24-42): the
    third slice (for v) is the identity rotation."""

    def __init__(self, seq_len: int, dim: int, base: float = 10_000.0):
        super().__init__()
        inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2) / dim))
        angles = torch.outer(torch.arange(seq_len).float(), inv_freq)
        angles = torch.cat((angles, angles), dim=-1)
        cos = angles.cos().view(1, seq_len, 1, 1, dim).repeat(1, 1, 3, 1, 1)
        sin = angles.sin().view(1, seq_len, 1, 1, dim).repeat(1, 1, 3, 1, 1)
        cos[:, :, 2] = 1.0
        sin[:, :, 2] = 0.0
        self.register_buffer("cos_cached", cos)
        self.register_buffer("sin_cached", sin)

    def forward(self) -> tuple[Tensor, Tensor]:
        return self.cos_cached, self.sin_cached

    def half_tables(self) -> tuple[Tensor, Tensor]:
        """``[S,D/2]`` tables of the q/k rotation."""
        half = self.cos_cached.shape[-1] // 2
        return self.cos_cached[0, :, 0, 0, :half], self.sin_cached[0, :, 0, 0, :half]


class TimestepEmbedder(nn.Module):
    """Sinusoidal features of a scalar time followed by a two-layer MLP (duo.py:68-93)."""

    def __init__(self, hidden_size: int, frequency_embedding_size: int = 256, max_period: float = 10000.0):
        super().__init__()
        self.mlp = nn.Sequential(
            nn.Linear(frequency_embedding_size, hidden_size),
            nn.SiLU(),
            nn.Linear(hidden_size, hidden_size),
        )
        half = frequency_embedding_size // 2
        self.register_buffer("freqs", torch.exp(-math.log(max_period) * torch.arange(half) / half))

    def forward(self, t: Tensor) -> Tensor:
        phase = t[:, None] * self.freqs[None, :]
        return self.mlp(torch.cat((phase.cos(), phase.sin()), dim=-1))


class DDiTBlock(nn.Module):
    """adaLN-modulated transformer block (duo.py:101-166)."""

    def __init__(self, dim: int, n_heads: int, seq_len: int, cond_dim: int, mlp_ratio: int = 4,
                 dropout: float = 0.1):
        super().__init__()
        self.n_heads, self.dim, self.seq_len = n_heads, dim, seq_len
        self.norm1 = nn.LayerNorm(dim)
        self.attn_qkv = nn.Linear(dim, 3 * dim, bias=False)
        self.attn_out = nn.Linear(dim, dim, bias=False)
        self.norm2 = nn.LayerNorm(dim)
        self.mlp = nn.Sequential(
            nn.Linear(dim, mlp_ratio * dim),
            nn.GELU(approximate="tanh"),
            nn.Linear(mlp_ratio * dim, dim),
        )
        self.dropout = nn.Dropout(dropout)
        self.adaLN_modulation = nn.Linear(cond_dim, 6 * dim)
        nn.init.zeros_(self.adaLN_modulation.weight)
        nn.init.zeros_(self.adaLN_modulation.bias)

    def forward(self, x: Tensor, cos: Tensor, sin: Tensor, c: Tensor,
                attention: Callable[[Tensor, Tensor, Tensor], Tensor], rotary_kernel: bool = False) -> Tensor:
        B = x.shape[0]
        shift_a, scale_a, gate_a, shift_m, scale_m, gate_m = self.adaLN_modulation(c)[:, None].chunk(6, dim=2)
        h = self.norm1(x) * (1.0 + scale_a) + shift_a
        qkv = self.attn_qkv(h).view(B, self.seq_len, 3, self.n_heads, self.dim // self.n_heads)
        v = qkv[:, :, 2]
        if rotary_kernel and attention is safe_sdpa_jvp:
            # the attention kernels read q, k, v (and their tangents) as strided views of the fused
            # projection and rotate q, k on chip; gradients come back through the inverse rotation
            # (shapes the folded rotation does not serve take the rotary kernel first)
            a = safe_sdpa_jvp_rotary(qkv[:, :, 0], qkv[:, :, 1], v, cos, sin)
            a = a.reshape(B, self.seq_len, self.dim)
            x = self.dropout(self.attn_out(a) * gate_a) + x
            h = self.norm2(x) * (1.0 + scale_m) + shift_m
            return self.dropout(self.mlp(h) * gate_m) + x
        if rotary_kernel:
            # one launch rotates q and k (and their tangents) out of the fused projection and writes
            # the contiguous 16-bit tensors the attention kernels read
            q, k = apply_rotary((qkv[:, :, 0], qkv[:, :, 1]), cos, sin)
        else:
            q = rotate_half_embedding(qkv[:, :, 0], cos, sin).contiguous()
            k = rotate_half_embedding(qkv[:, :, 1], cos, sin).contiguous()
        # v stays a strided view of the fused projection: the attention kernels read through strides
        a = attention(q, k, v if rotary_kernel else v.contiguous())  # [B,S,H,D] (duo.py:141)
        a = a.reshape(B, self.seq_len, self.dim)
        x = self.dropout(self.attn_out(a) * gate_a) + x
        h = self.norm2(x) * (1.0 + scale_m) + shift_m
        return self.dropout(self.mlp(h) * gate_m) + x


class EmbeddingLayer(nn.Module):
    """Linear map from the (relaxed one-hot) vocabulary axis to the model width (duo.py:169-180)."""

    def __init__(self, dim: int, vocab_dim: int):
        super().__init__()
        self.seq = nn.Linear(vocab_dim, dim)
        self._coeff = vocab_dim ** 0.5

    def forward(self, x: Tensor) -> Tensor:
        return self.seq(x / self._coeff)


class DDiTFinalLayer(nn.Module):
    """adaLN-modulated LayerNorm and projection back to the vocabulary (duo.py:183-202)."""

    def __init__(self, hidden_size: int, out_channels: int, cond_dim: int):
        super().__init__()
        self.norm_final = nn.LayerNorm(hidden_size)
        self.linear = nn.Linear(hidden_size, out_channels)
        self.adaLN_modulation = nn.Linear(cond_dim, 2 * hidden_size)
        for lin in (self.linear, self.adaLN_modulation):
            nn.init.zeros_(lin.weight)
            nn.init.zeros_(lin.bias)

    def forward(self, x: Tensor, c: Tensor) -> Tensor:
        shift, scale = self.adaLN_modulation(c)[:, None].chunk(2, dim=2)
        return self.linear(self.norm_final(x) * (1.0 + scale) + shift)


class DIT(nn.Module):
    """``net(x, s, t, jvp_attention=False) -> logits`` with ``x`` ``[B,S,V]`` and ``s, t`` ``[B]``
    (duo.py:299-360; the "naive" input embedding, which is what the text configurations use).

    ``jvp_attention=True`` routes attention through the fused attention-JVP op, which is what lets
    ``torch.func.jvp`` run over the network.  With ``jvp_attention=False`` the reference calls
    ``F.scaled_dot_product_attention`` (duo.py:143-152); ``plain_attention`` selects that ("torch") or
    the primal-only mode of the same HIP kernels ("hip", the default).  ``attention_override`` replaces
    both with a caller-supplied function of ``(q, k, v)`` in ``[B,S,H,D]`` (the tests use
    :func:`math_attention`).  ``rotary`` selects the rotary embedding of q and k: "hip" (one launch
    of the library's rotary kernel per block; GPU tensors only, there is no fallback) or "torch"
    (:func:`rotate_half_embedding`, the separate PyTorch operations of the reference).
    """

    def __init__(self, vocab_size: int, hidden_size: int, cond_dim: int, n_blocks: int, n_heads: int,
                 dropout: float, length: int, plain_attention: str = "hip",
                 attention_override: Optional[Callable[[Tensor, Tensor, Tensor], Tensor]] = None,
                 rotary: str = "hip"):
        super().__init__()
        if plain_attention not in ("hip", "torch"):
            raise ValueError(f"illegal 'plain_attention': {plain_attention}")
        self.vocab_size = vocab_size
        if rotary not in ("hip", "torch"):
            raise ValueError(f"illegal 'rotary': {rotary}")
        self.plain_attention = plain_attention
        self.attention_override = attention_override
        self.rotary = rotary
        self.vocab_embed = EmbeddingLayer(hidden_size, vocab_size)
        self.s_map = TimestepEmbedder(cond_dim)
        self.t_map = TimestepEmbedder(cond_dim)
        self.rotary_emb = Rotary(length, hidden_size // n_heads)
        self.blocks = nn.ModuleList(
            DDiTBlock(hidden_size, n_heads, length, cond_dim, dropout=dropout) for _ in range(n_blocks))
        self.output_layer = DDiTFinalLayer(hidden_size, vocab_size, cond_dim)

    @staticmethod
    def _torch_attention(q: Tensor, k: Tensor, v: Tensor) -> Tensor:
        out = F.scaled_dot_product_attention(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2))
        return out.transpose(1, 2)

    def _attention(self, jvp_attention: bool) -> Callable[[Tensor, Tensor, Tensor], Tensor]:
        if self.attention_override is not None:
            return self.attention_override
        if jvp_attention or self.plain_attention == "hip":
            return safe_sdpa_jvp
        return self._torch_attention

    def forward(self, x: Tensor, s: Tensor, t: Tensor, jvp_attention: bool = False) -> Tensor:
        t = t - s  # the network is conditioned on the start time and the time span (duo.py:346-351)
        cond = F.silu(self.s_map(s)) + F.silu(self.t_map(t))
        h = self.vocab_embed(x)
        cos, sin = self.rotary_emb.half_tables()
        attention = self._attention(jvp_attention)
        rotary_kernel = self.rotary == "hip"
        for block in self.blocks:
            h = block(h, cos, sin, cond, attention, rotary_kernel)
        return self.output_layer(h, cond)
