"""CPU oracle of the routed-expert FFN forward.  TEST INFRASTRUCTURE ONLY.

Restates, in fp32 on dequantised operands, the three device stages the reference
chains for one forward step (campaigns/mok/port/framework/interp_fwd.cu:174-213):

1. routed gate / routed up grouped GEMM   (campaigns/mok/port/gemm/gemm.cu:150-157)
     gate[r,:] = sum_k deq(x[row_token[r],k]) * deq(Wg[e(r)][:,k]),  same for up
2. clamped SwiGLU, rounded to bf16, then MXFP8 requant along the d_ff axis
     (campaigns/mok/port/act_gptoss/swiglu.cuh:157-187,
      campaigns/mok/host/act_gptoss_reference.py:16-21)
3. routed down grouped GEMM -> bf16        (campaigns/mok/port/gemm/gemm.cu:158-162)
     y[r,:] = sum_k deq(hidden[r,k]) * deq(Wd[e(r)][:,k])

Weights are ``[E, N, K]`` (N x K row-major, the reference's "column-major B",
campaigns/mok/port/gemm/provider.cu:79-82).  Rows are grouped by expert; expert e owns
rows ``[offsets[e], offsets[e+1])``.
"""
from __future__ import annotations

import numpy as np
import torch

from . import mxfp8

SWIGLU_ALPHA = 1.702  # campaigns/mok/port/act_gptoss/swiglu.cuh:2


def route_topk(logits: torch.Tensor, k: int) -> torch.Tensor:
    """Expert ids ``[T, k]``: top-k of softmax(logits) (campaigns/mok/host/mok_port_host.py:273-282)."""
    p = torch.softmax(logits.float(), dim=-1)
    return torch.topk(p, k, dim=-1).indices


def group_rows(idx: np.ndarray, num_experts: int):
    """Stable sort of the (token, slot) pairs by expert id.

    Returns (tokens_per_expert[E] int32, row_token[R] int32, row_slot[R] int32)."""
    idx = np.asarray(idx)
    t, k = idx.shape
    flat = idx.reshape(-1)
    order = np.argsort(flat, kind="stable")
    counts = np.bincount(flat, minlength=num_experts).astype(np.int32)
    return counts, (order // k).astype(np.int32), (order % k).astype(np.int32)


def gptoss_swiglu(gate: np.ndarray, up: np.ndarray, limit: float | None, alpha: float = SWIGLU_ALPHA) -> np.ndarray:
    """(up + 1) * gate * sigmoid(alpha * gate) with gate <= limit, |up| <= limit, in fp32."""
    g = np.asarray(gate, dtype=np.float32)
    u = np.asarray(up, dtype=np.float32)
    if limit is not None:
        lim = np.float32(limit)
        g = np.minimum(g, lim)
        u = np.clip(u, -lim, lim)
    sig = (np.float32(1.0) / (np.float32(1.0) + np.exp(-np.float32(alpha) * g))).astype(np.float32)
    return ((u + np.float32(1.0)) * (g * sig)).astype(np.float32)


def grouped_matmul(a: np.ndarray, w: np.ndarray, counts: np.ndarray) -> np.ndarray:
    """out[r,:] = a[r,:] @ w[e(r)].T in fp32, rows grouped by expert.  a [R,K], w [E,N,K]."""
    r_total = int(np.sum(counts))
    out = np.zeros((r_total, w.shape[1]), dtype=np.float32)
    off = 0
    for e, c in enumerate(np.asarray(counts).tolist()):
        if c:
            at = torch.from_numpy(np.ascontiguousarray(a[off:off + c]))
            wt = torch.from_numpy(np.ascontiguousarray(w[e]))
            out[off:off + c] = torch.matmul(at, wt.t()).numpy()
        off += c
    return out


def grouped_matmul_naive(a: np.ndarray, w: np.ndarray, counts: np.ndarray) -> np.ndarray:
    """Triple-loop version in float64 for tiny shapes (the brute-force check of grouped_matmul)."""
    r_total = int(np.sum(counts))
    n, k = w.shape[1], w.shape[2]
    out = np.zeros((r_total, n), dtype=np.float64)
    r = 0
    for e, c in enumerate(np.asarray(counts).tolist()):
        for _ in range(c):
            for j in range(n):
                s = 0.0
                for kk in range(k):
                    s += float(a[r, kk]) * float(w[e, j, kk])
                out[r, j] = s
            r += 1
    return out


def moe_ffn_forward(x_q, x_sc, wg_q, wg_sc, wu_q, wu_sc, wd_q, wd_sc, counts, row_token,
                    limit: float | None = 7.0, alpha: float = SWIGLU_ALPHA):
    """Whole routed forward on pre-quantised bytes.

    x_q [T,H] u8 / x_sc [T,ld];  w*_q [E,N,K] u8 / w*_sc [E,N,ld];  counts [E];  row_token [R].
    Returns dict(y_bf16_bits u16 [R,H], y f32, hidden_q, hidden_sc, hidden f32 (bf16-rounded, pre-quant))."""
    x = mxfp8.mx_dequantize(x_q, x_sc)
    a = x[np.asarray(row_token)]
    e_count = wg_q.shape[0]
    gate = np.zeros((a.shape[0], wg_q.shape[1]), dtype=np.float32)
    up = np.zeros_like(gate)
    off = 0
    for e in range(e_count):
        c = int(counts[e])
        if c:
            one = np.zeros(e_count, dtype=np.int64)
            one[e] = c
            wg = mxfp8.mx_dequantize(wg_q[e:e + 1], wg_sc[e:e + 1])
            wu = mxfp8.mx_dequantize(wu_q[e:e + 1], wu_sc[e:e + 1])
            gate[off:off + c] = grouped_matmul(a[off:off + c], wg, [c])
            up[off:off + c] = grouped_matmul(a[off:off + c], wu, [c])
        off += c
    hidden = mxfp8.bf16_round(gptoss_swiglu(gate, up, limit, alpha))  # swiglu.cuh:175 rounds to bf16 first
    hidden_q, hidden_sc = mxfp8.mx_quantize(hidden)
    hd = mxfp8.mx_dequantize(hidden_q, hidden_sc)
    y = np.zeros((a.shape[0], wd_q.shape[1]), dtype=np.float32)
    off = 0
    for e in range(e_count):
        c = int(counts[e])
        if c:
            wd = mxfp8.mx_dequantize(wd_q[e:e + 1], wd_sc[e:e + 1])
            y[off:off + c] = grouped_matmul(hd[off:off + c], wd, [c])
        off += c
    return {
        "y": mxfp8.bf16_round(y),
        "y_bf16_bits": mxfp8.bf16_bits(y),
        "hidden": hidden,
        "hidden_q": hidden_q,
        "hidden_sc": hidden_sc,
        "gate": gate,
        "up": up,
    }


def rel_frobenius(got: np.ndarray, ref: np.ndarray) -> float:
    """||got - ref||_F / ||ref||_F in float64."""
    g = np.asarray(got, dtype=np.float64)
    r = np.asarray(ref, dtype=np.float64)
    den = float(np.sqrt(np.sum(r * r)))
    return float(np.sqrt(np.sum((g - r) ** 2)) / den) if den else float(np.sqrt(np.sum(g * g)))


# ---- the same pipeline in torch ops (multi-threaded; what bench.py times as the CPU baseline) ----
def _deq_torch(q: torch.Tensor, sc: torch.Tensor) -> torch.Tensor:
    k = q.shape[-1]
    nb = k // mxfp8.MX_BLOCK
    vals = q.contiguous().view(torch.float8_e4m3fn).float().reshape(q.shape[:-1] + (nb, mxfp8.MX_BLOCK))
    scale = ((sc[..., :nb].to(torch.int32)) << 23).view(torch.float32)  # 2**(b-127) for 1 <= b <= 254
    scale = torch.where(sc[..., :nb] == 0, torch.full_like(scale, 2.0 ** -127), scale)
    return (vals * scale.unsqueeze(-1)).reshape(q.shape)


def _quant_torch(x: torch.Tensor):
    nb = x.shape[-1] // mxfp8.MX_BLOCK
    blk = x.reshape(x.shape[:-1] + (nb, mxfp8.MX_BLOCK))
    amax = blk.abs().amax(dim=-1)
    b = (((amax.view(torch.int32) >> 23) & 0xFF) - 8).clamp_(0, 254)
    inv = ((254 - b) << 23).view(torch.float32)
    codes = (blk * inv.unsqueeze(-1)).clamp_(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    return codes.reshape(x.shape), b.to(torch.uint8)


def moe_ffn_forward_torch(x_q, x_sc, wg_q, wg_sc, wu_q, wu_sc, wd_q, wd_sc, counts, row_token,
                          limit: float | None = 7.0, alpha: float = SWIGLU_ALPHA) -> torch.Tensor:
    """Same arithmetic as ``moe_ffn_forward`` with torch kernels; returns y as bf16 [R, H]."""
    a = _deq_torch(x_q, x_sc)[row_token.long()]
    rows = a.shape[0]
    hidden = torch.empty((rows, wg_q.shape[1]), dtype=torch.float32)
    off = 0
    for e, c in enumerate(counts.tolist()):
        if c:
            ae = a[off:off + c]
            g = ae @ _deq_torch(wg_q[e], wg_sc[e]).t()
            u = ae @ _deq_torch(wu_q[e], wu_sc[e]).t()
            if limit is not None:
                g = g.clamp(max=limit)
                u = u.clamp(min=-limit, max=limit)
            hidden[off:off + c] = ((u + 1.0) * (g * torch.sigmoid(alpha * g))).to(torch.bfloat16).float()
        off += c
    hq, hb = _quant_torch(hidden)
    hd = _deq_torch(hq, hb)
    y = torch.empty((rows, wd_q.shape[1]), dtype=torch.float32)
    off = 0
    for e, c in enumerate(counts.tolist()):
        if c:
            y[off:off + c] = hd[off:off + c] @ _deq_torch(wd_q[e], wd_sc[e]).t()
        off += c
    return y.to(torch.bfloat16)
