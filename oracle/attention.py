"""CPU oracle of the flash-attention prefill example.  TEST INFRASTRUCTURE ONLY.

softmax(scale * Q K^T + causal mask) V per query head in fp32, grouped-query (query head h reads KV head
h // (Hq / Hkv)), as the reference's attention campaign defines its dense causal workload
(campaigns/attention/README.md:118-128: bf16, head dimension 128, scale 1 / sqrt(128)).

Pins: ``attention_head`` (restated with explicit matmul / softmax) against torch's
``scaled_dot_product_attention`` (library routine); closed forms -- the first query only sees key 0, so
its output is V[0]; with all keys equal the output is the running mean of V.
"""
from __future__ import annotations

import math

import torch


def inputs(batch: int, q_heads: int, kv_heads: int, seq: int, dim: int = 128, seed: int = 0):
    """(Q [B,Hq,S,D], K, V [B,Hkv,S,D]) bf16 from N(0,1); draw order Q, K, V."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(batch, q_heads, seq, dim, generator=g).to(torch.bfloat16)
    k = torch.randn(batch, kv_heads, seq, dim, generator=g).to(torch.bfloat16)
    v = torch.randn(batch, kv_heads, seq, dim, generator=g).to(torch.bfloat16)
    return q, k, v


def attention_head(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float | None = None, window: int | None = None) -> torch.Tensor:
    """One head: q, k, v [S, D] -> [S, D] fp32, causal; with `window`, a query sees only the last `window` keys up to
    its own (campaigns/attention/src/sm90/stage_mask_window.cu: kv_pos > q_pos - window)."""
    s, d = q.shape
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    scores = (q.float() @ k.float().t()) * scale
    hidden = torch.ones(s, s, dtype=torch.bool).triu(1)
    if window is not None:
        hidden |= torch.ones(s, s, dtype=torch.bool).tril(-window)
    scores = scores.masked_fill(hidden, float("-inf"))
    return torch.softmax(scores, dim=-1) @ v.float()


def attention_head_library(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    return torch.nn.functional.scaled_dot_product_attention(q.float()[None], k.float()[None], v.float()[None], is_causal=True)[0]


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, heads: list[tuple[int, int]] | None = None,
              window: int | None = None) -> dict[tuple[int, int], torch.Tensor]:
    """{(batch, query head): [S, D] fp32} for the listed heads (all if None)."""
    b, hq, _, _ = q.shape
    group = hq // k.shape[1]
    heads = [(i, h) for i in range(b) for h in range(hq)] if heads is None else heads
    return {(i, h): attention_head(q[i, h], k[i, h // group], v[i, h // group], window=window) for i, h in heads}
