"""CPU oracle of the decode megakernel example: one decoding step of a Llama-shaped model in fp32.
TEST INFRASTRUCTURE ONLY.

Per layer: RMSNorm -> fused QKV matvec -> rotary embedding (rotate-half pairing, element i with i + 32) ->
append the rotated key and the value to the bf16 cache -> softmax attention of every query head over its KV
head's cache (grouped-query) -> output projection + residual -> RMSNorm -> silu(gate) * up -> down projection
+ residual; then the final RMSNorm and the LM head (campaigns/megakernel in the reference runs the same op
list as one persistent kernel: port/src/ops/{qkv,attn_partial,attn_reduction,o_proj,upgate,down_proj,lm_head}.cu).
Weights and cache are bf16; activations fp32.

Pins: ``rms_norm`` against torch.nn.functional.rms_norm; the attention against
scaled_dot_product_attention; ``silu`` against torch.nn.functional.silu; rotary embedding by its invariants
(norm preserved; q_m . k_n depends on m - n only).
"""
from __future__ import annotations

import math

import numpy as np
import torch

HEAD_DIM = 64


def layer_views(weights: torch.Tensor, layer: int, d: int, hq: int, hkv: int, dff: int) -> dict[str, torch.Tensor]:
    """Views into the packed bf16 weights (as the kernel reads them, pipelink_amd/stages/megakernel/include/mk_abi.h)."""
    qkv, od = (hq + 2 * hkv) * HEAD_DIM, hq * HEAD_DIM
    per = d + qkv * d + d * od + d + 2 * dff * d + d * dff
    p = weights[layer * per:(layer + 1) * per]
    out, o = {}, 0
    for name, shape in (("attn_norm", (d,)), ("wqkv", (qkv, d)), ("wo", (d, od)), ("ffn_norm", (d,)), ("wgate", (dff, d)),
                        ("wup", (dff, d)), ("wdown", (d, dff))):
        n = int(np.prod(shape))
        out[name] = p[o:o + n].view(shape)
        o += n
    return out


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt((x * x).mean() + eps) * w.float()


def rope(v: torch.Tensor, pos: int, theta: float = 500000.0) -> torch.Tensor:
    """v [..., 64]; element i pairs with i + 32."""
    inv = theta ** (-torch.arange(0, HEAD_DIM, 2, dtype=torch.float64) / HEAD_DIM)
    ang = pos * inv
    c, s = torch.cos(ang).float(), torch.sin(ang).float()
    a, b = v[..., :32], v[..., 32:]
    return torch.cat([a * c - b * s, b * c + a * s], dim=-1)


def silu(x: torch.Tensor) -> torch.Tensor:
    return x / (1.0 + torch.exp(-x))


def decode_step(weights: torch.Tensor, kv_cache: torch.Tensor, x: torch.Tensor, *, layers: int, d: int, hq: int, hkv: int, dff: int,
                vocab: int, pos: int, eps: float = 1e-5):
    """weights: packed bf16 tensor; kv_cache bf16 [L, 2, smax, hkv, 64] (positions < pos filled; updated in place
    at `pos`); x fp32 [d].  Returns (logits [vocab] fp32, x after the last layer)."""
    x = x.clone().float()
    group = hq // hkv
    for l in range(layers):
        w = layer_views(weights, l, d, hq, hkv, dff)
        qkv = w["wqkv"].float() @ rms_norm(x, w["attn_norm"], eps)
        q = rope(qkv[:hq * HEAD_DIM].view(hq, HEAD_DIM), pos)
        k = rope(qkv[hq * HEAD_DIM:(hq + hkv) * HEAD_DIM].view(hkv, HEAD_DIM), pos)
        v = qkv[(hq + hkv) * HEAD_DIM:].view(hkv, HEAD_DIM)
        kv_cache[l, 0, pos] = k.to(torch.bfloat16)
        kv_cache[l, 1, pos] = v.to(torch.bfloat16)
        keys = kv_cache[l, 0, :pos + 1].float()    # [pos+1, hkv, 64]
        vals = kv_cache[l, 1, :pos + 1].float()
        att = torch.empty(hq, HEAD_DIM)
        for h in range(hq):
            s = (keys[:, h // group] @ q[h]) / math.sqrt(HEAD_DIM)
            att[h] = torch.softmax(s, dim=0) @ vals[:, h // group]
        x = x + w["wo"].float() @ att.reshape(-1)
        hn = rms_norm(x, w["ffn_norm"], eps)
        x = x + w["wdown"].float() @ (silu(w["wgate"].float() @ hn) * (w["wup"].float() @ hn))
    per = layers * (d + (hq + 2 * hkv) * HEAD_DIM * d + d * hq * HEAD_DIM + d + 2 * dff * d + d * dff)
    final_norm, lm = weights[per:per + d], weights[per + d:per + d + vocab * d].view(vocab, d)
    logits = torch.empty(vocab)
    xn = rms_norm(x, final_norm, eps)
    for r0 in range(0, vocab, 16384):    # in pieces: the fp32 copy of the LM head would be 1 GB
        logits[r0:r0 + 16384] = lm[r0:r0 + 16384].float() @ xn
    return logits, x


def make_model(*, layers: int, d: int, hq: int, hkv: int, dff: int, vocab: int, pos: int, smax: int, seed: int = 0):
    """(packed bf16 weights from N(0,1) * 0.02 -- norm weights 1 + N(0,1) * 0.02 --, bf16 cache with positions < pos from
    N(0,1), x [d] fp32 from N(0,1))."""
    g = torch.Generator().manual_seed(seed)
    qkv, od = (hq + 2 * hkv) * HEAD_DIM, hq * HEAD_DIM
    parts = []

    def mat(n):   # in pieces, to bound the fp32 temporary
        for s in range(0, n, 1 << 26):
            parts.append((torch.randn(min(1 << 26, n - s), generator=g) * 0.02).to(torch.bfloat16))

    def norm(n):
        parts.append((1.0 + torch.randn(n, generator=g) * 0.02).to(torch.bfloat16))

    for _ in range(layers):
        norm(d); mat(qkv * d); mat(d * od); norm(d); mat(dff * d); mat(dff * d); mat(d * dff)
    norm(d); mat(vocab * d)
    weights = torch.cat(parts)
    cache = torch.zeros(layers, 2, smax, hkv, HEAD_DIM, dtype=torch.bfloat16)
    cache[:, :, :pos] = torch.randn(layers, 2, pos, hkv, HEAD_DIM, generator=g).to(torch.bfloat16)
    x = torch.randn(d, generator=g)
    return weights, cache, x
