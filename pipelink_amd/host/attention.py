"""Host side of the flash-attention prefill example on the host-less route."""
from __future__ import annotations

from pathlib import Path

import numpy as np

from ..pipec.launcher import HostlessSession, open_hostless
from ..stages.attention.params import params_blobs

HEAD_DIM = 128
Q_TILE = 128


def open_session(link_json: str | Path, q_bits: np.ndarray, k_bits: np.ndarray, v_bits: np.ndarray, *, scale: float | None = None,
                 window: int | None = None, backend=None, image: str | Path | None = None) -> HostlessSession:
    """q_bits [B, Hq, S, 128], k_bits / v_bits [B, Hkv, S, 128]: bf16 bit patterns (uint16).  Buffers: q, k, v and
    o ([B, S, Hq * 128] uint16, zeroed).  `window`: for a link with fa.mask.window, the number of keys a query sees.
    (A link names one mask package; the params blob must be addressed to it.)"""
    if window is not None and window < 1:
        raise ValueError("a window is at least one key")
    if scale is not None and not (np.isfinite(scale) and scale > 0):
        raise ValueError("the softmax scale must be a positive finite number (masked scores are -1e30 times it)")
    if q_bits.ndim != 4 or k_bits.shape != v_bits.shape or k_bits.ndim != 4:
        raise ValueError("q is [B, Hq, S, D]; k and v are [B, Hkv, S, D]")
    b, hq, s, d = q_bits.shape
    b2, hkv, s2, d2 = k_bits.shape
    if (b, s, d) != (b2, s2, d2) or d != HEAD_DIM or s % Q_TILE or hkv <= 0 or hq % hkv:
        raise ValueError("head dimension must be 128, the sequence a multiple of 128, query heads a multiple of KV heads")
    if any(t.dtype != np.uint16 for t in (q_bits, k_bits, v_bits)):
        raise ValueError("operands are uint16 bf16 bit patterns")
    if s * d * 2 >= 1 << 31:
        raise ValueError("one head of K or V must stay below 2 GiB")
    buffers = {"q": q_bits, "k": k_bits, "v": v_bits, "o": ((b, s, hq * d), np.uint16)}
    return open_hostless(link_json, buffers=buffers, params=lambda addr: params_blobs(addr, b, hq, hkv, s, scale, window),
                         grid=(b * hq * (s // Q_TILE),), backend=backend, image=image)
