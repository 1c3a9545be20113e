"""Seeded synthetic inputs of the routed-expert FFN forward.

Draw order (CPU generator, seed given): router logits [T,E], x [T,H], then gate, up and
down weights [E,N,K] scaled by 0.02, one expert at a time.  Routing is top-k of
softmax(logits); the (token, slot) pairs are stably sorted by expert, which gives the
routed-row order, ``tokens_per_expert`` and ``row_token``.  Follows the style of
``MoKHost.new_inputs`` (campaigns/mok/host/mok_port_host.py:273-282), including its
concentrated-routing generations that leave experts empty."""
from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import mxfp8


@dataclass
class MokInputs:
    tokens_per_expert: torch.Tensor  # [E] int32
    row_token: torch.Tensor          # [R] int32
    x_q: torch.Tensor
    x_sc: torch.Tensor
    w_gate_q: torch.Tensor
    w_gate_sc: torch.Tensor
    w_up_q: torch.Tensor
    w_up_sc: torch.Tensor
    w_down_q: torch.Tensor
    w_down_sc: torch.Tensor

    def to(self, device):
        return MokInputs(**{k: v.to(device) for k, v in self.__dict__.items()})


def route(logits: torch.Tensor, top_k: int):
    idx = torch.topk(torch.softmax(logits.float(), dim=-1), top_k, dim=-1).indices
    flat = idx.reshape(-1)
    order = torch.sort(flat, stable=True).indices
    counts = torch.bincount(flat, minlength=logits.shape[1]).to(torch.int32)
    return counts, (order // top_k).to(torch.int32)


def generate(num_tokens: int, hidden: int, intermediate: int, num_experts: int, top_k: int, seed: int = 0,
             concentrate: int = 0, quantize_device: torch.device | None = None,
             counts: list[int] | None = None) -> MokInputs:
    """``concentrate`` > 0 routes every token to the first ``concentrate`` experts only (empty experts).
    ``counts`` sets the experts' row counts directly (``top_k`` is then unused): every routed row reads a token
    drawn at random."""
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(num_tokens, num_experts, generator=g)
    if concentrate:
        logits[:, concentrate:] = -1e9
    x = torch.randn(num_tokens, hidden, generator=g)
    if counts is not None:
        if len(counts) != num_experts:
            raise ValueError("counts must give one row count per expert")
        row_token = torch.randint(num_tokens, (sum(counts),), generator=g).to(torch.int32)
        counts = torch.tensor(counts, dtype=torch.int32)
    else:
        counts, row_token = route(logits, top_k)
    dev = quantize_device or torch.device("cpu")
    x_q, x_sc = mxfp8.quantize(x.to(dev))

    def weights(n, k):
        qs, scs = [], []
        for _ in range(num_experts):
            w = torch.randn(n, k, generator=g) * 0.02
            q, sc = mxfp8.quantize(w.to(dev))
            qs.append(q)
            scs.append(sc)
        return torch.stack(qs), torch.stack(scs)

    wg_q, wg_sc = weights(intermediate, hidden)
    wu_q, wu_sc = weights(intermediate, hidden)
    wd_q, wd_sc = weights(hidden, intermediate)
    return MokInputs(counts.to(dev), row_token.to(dev), x_q, x_sc, wg_q, wg_sc, wu_q, wu_sc, wd_q, wd_sc)


# ---- result checks of the harness ------------------------------------------------------------------------
# The reference's host harness reports three global error figures and a pass rule on two of them
# (campaigns/mok/host/mok_port_host.py:291-314) and compares images byte for byte (:317-320).  Its
# tolerance constants live in the absent upstream package; the one pair visible in the reference is the
# bf16 one quoted in campaigns/mok/evidence/REPORT.md:22.
BF16_TOLERANCE = (5e-1, 1e-2)  # (absolute on the largest error, relative on sum|err| / sum|ref|)


def error_stats(expected, actual, chunk: int = 1 << 26) -> tuple[float, float, float]:
    """(mean |err|, max |err|, sum|err| / sum|ref|) over all elements, accumulated in float64 over
    chunks so that the fp32 copies stay bounded."""
    import numpy as np

    e = np.asarray(expected).reshape(-1)
    a = np.asarray(actual).reshape(-1)
    if e.shape != a.shape:
        raise ValueError("expected and actual differ in size")
    abs_sum = ref_sum = 0.0
    maximum = 0.0
    for start in range(0, e.size, chunk):
        ref = e[start:start + chunk].astype(np.float32)
        diff = np.abs(ref - a[start:start + chunk].astype(np.float32))
        abs_sum += float(diff.sum(dtype=np.float64))
        ref_sum += float(np.abs(ref).sum(dtype=np.float64))
        maximum = max(maximum, float(diff.max())) if diff.size else maximum
    n = max(e.size, 1)
    return abs_sum / n, maximum, (abs_sum / ref_sum if ref_sum else float("inf") if abs_sum else 0.0)


def tolerance_report(expected, actual, tolerance: tuple[float, float] = BF16_TOLERANCE) -> dict:
    import math

    mean, maximum, relative = error_stats(expected, actual)
    atol, rtol = tolerance
    return dict(abs_mean=mean, abs_max=maximum, relative=relative, absolute_tolerance=atol, relative_tolerance=rtol,
                passed=all(math.isfinite(v) for v in (mean, maximum, relative)) and maximum <= atol and relative <= rtol)


def bitwise_report(left, right) -> bool:
    """Byte equality of two tensors or arrays of the same layout."""
    import numpy as np

    def raw(t):
        if isinstance(t, torch.Tensor):
            return t.detach().cpu().contiguous().view(torch.uint8).numpy()
        return np.ascontiguousarray(t).view(np.uint8)
    l, r = raw(left), raw(right)
    return l.shape == r.shape and bool(np.array_equal(l, r))
