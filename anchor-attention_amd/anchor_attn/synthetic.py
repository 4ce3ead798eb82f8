"""Seeded synthetic long-context q/k/v for the AnchorAttention prefill operator.

The tensors have the statistics the operator is designed for: i.i.d. N(0,1) queries and keys
with rotary position embedding applied, an attention sink at key 0 and a sparse set of "stripe"
keys that every later query attends to.  Sink and stripes are produced by adding multiples of a
per-KV-head vector ``qbar`` to those keys:

* ``qbar_mode="shared"`` (default): ``qbar`` is a seeded random direction of squared norm
  ``16 / (4 * sm_scale)`` (45.25 for D=128) that is also added to every query of the KV group
  after RoPE, so the sink scores about +16 nats and a stripe about +8 nats above ordinary keys.
* ``qbar_mode="literal"``: ``qbar`` is the sample mean of the group's RoPE'd queries; its norm is
  about ``sqrt(D/N)``, the biases are negligible and the operator runs in its dense regime.

Everything is generated on the CPU with one ``torch.Generator`` so that a CPU checker and the GPU
see bit-identical inputs; ``device`` only says where the result is moved to.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


def rope_rotate_half(x: torch.Tensor, base: float) -> torch.Tensor:
    """Rotate-half RoPE at positions ``0..N-1`` on a ``[..., N, D]`` float32 tensor."""
    n, d = x.shape[-2], x.shape[-1]
    inv_freq = 1.0 / (base ** (torch.arange(0, d, 2, dtype=torch.float64) / d))
    ang = torch.arange(n, dtype=torch.float64)[:, None] * inv_freq[None, :]
    cos = torch.cat([ang.cos(), ang.cos()], dim=-1).to(torch.float32)
    sin = torch.cat([ang.sin(), ang.sin()], dim=-1).to(torch.float32)
    x1, x2 = x[..., : d // 2], x[..., d // 2 :]
    rot = torch.cat([-x2, x1], dim=-1)
    return x * cos + rot * sin


def stripe_positions(n_ctx: int, n_stripes: int, dist: str, gen: torch.Generator) -> torch.Tensor:
    """``n_stripes`` distinct key positions in ``[1, n_ctx)`` (position 0 is the sink).

    ``dist="uniform"`` draws uniformly; ``dist="powerlaw"`` draws position ``x`` with density
    proportional to ``x**-0.5`` (inverse-CDF ``x = 1 + (n_ctx-2) * u**2``), so stripes thin out
    with distance from the start of the context."""
    if n_stripes <= 0:
        return torch.zeros(0, dtype=torch.long)
    if dist == "uniform":
        perm = torch.randperm(n_ctx - 1, generator=gen)[:n_stripes] + 1
        return perm.sort().values
    if dist == "powerlaw":
        got = torch.zeros(0, dtype=torch.long)
        while got.numel() < n_stripes:
            u = torch.rand(4 * n_stripes, generator=gen, dtype=torch.float64)
            x = (1 + (n_ctx - 2) * u * u).floor().long().clamp_(1, n_ctx - 1)
            got = torch.unique(torch.cat([got, x]))
            if got.numel() > n_stripes:
                keep = torch.randperm(got.numel(), generator=gen)[:n_stripes]
                got = got[keep]
        return got.sort().values
    raise ValueError(f"unknown stripe distribution {dist!r}")


def make_qkv(
    n_ctx: int,
    n_q_heads: int = 32,
    n_kv_heads: int = 8,
    head_dim: int = 128,
    rope_base: float = 500000.0,
    n_stripes: int = 64,
    stripe_dist: str = "uniform",
    seed: int = 0,
    qbar_mode: str = "shared",
    dtype: torch.dtype = torch.bfloat16,
    device: Optional[str] = None,
    sink_gain: float = 4.0,
    stripe_gain: float = 2.0,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """Returns ``(q [1,Hq,N,D], k [1,Hkv,N,D], v [1,Hkv,N,D], stripe positions)``."""
    assert n_q_heads % n_kv_heads == 0
    group = n_q_heads // n_kv_heads
    gen = torch.Generator(device="cpu").manual_seed(seed)
    q = torch.randn(1, n_q_heads, n_ctx, head_dim, generator=gen, dtype=torch.float32)
    k = torch.randn(1, n_kv_heads, n_ctx, head_dim, generator=gen, dtype=torch.float32)
    v = torch.randn(1, n_kv_heads, n_ctx, head_dim, generator=gen, dtype=torch.float32)
    for h in range(n_q_heads):  # head by head keeps the float64 angle table small
        q[0, h] = rope_rotate_half(q[0, h], rope_base)
    for h in range(n_kv_heads):
        k[0, h] = rope_rotate_half(k[0, h], rope_base)
    pos = stripe_positions(n_ctx, n_stripes, stripe_dist, gen)
    if qbar_mode == "shared":
        sm_scale = 1.0 / math.sqrt(head_dim)
        norm2 = 16.0 / (4.0 * sm_scale)
        u = torch.randn(n_kv_heads, head_dim, generator=gen, dtype=torch.float32)
        qbar = u / u.norm(dim=-1, keepdim=True) * math.sqrt(norm2)
        q += qbar.repeat_interleave(group, dim=0)[None, :, None, :]
    elif qbar_mode == "literal":
        qbar = q[0].reshape(n_kv_heads, group * n_ctx, head_dim).mean(dim=1)
    else:
        raise ValueError(f"unknown qbar_mode {qbar_mode!r}")
    k[0, :, 0, :] += sink_gain * qbar
    if pos.numel():
        k[0, :, pos, :] += stripe_gain * qbar[:, None, :]
    q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
    if device is not None:
        q, k, v = q.to(device), k.to(device), v.to(device)
    return q, k, v, pos
