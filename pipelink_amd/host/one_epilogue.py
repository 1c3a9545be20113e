"""Host side of the one-epilogue-many-producers example (C = (A . B) * scale[col] + bias[col]) on the
host-less route: the same buffers and params for each of the linked pipelines (accumulator in AGPRs,
VGPRs, LDS with 128 x 128 workgroup tiles; `wide`: 256 x 128 tiles, accumulator in AGPRs) and their one-unit controls."""
from __future__ import annotations

from pathlib import Path

import numpy as np

from ..pipec.launcher import HostlessSession, open_hostless
from ..stages.one_epilogue.params import params_blobs

TILE = 128
TILE_K = 64


def open_session(link_json: str | Path, home: str, a_bits: np.ndarray, bt_bits: np.ndarray, bias: np.ndarray,
                 scale: np.ndarray, *, backend=None, image: str | Path | None = None) -> HostlessSession:
    """a_bits [m,k], bt_bits [n,k]: bf16 bit patterns (uint16); bias, scale [n] float32.  Buffers: a, bt, bias,
    scale, c ([m,n] uint16, zeroed), status ([1] uint32: non-zero if a ring wait gave up)."""
    m, k = a_bits.shape
    n, k2 = bt_bits.shape
    if k != k2 or bias.shape != (n,) or scale.shape != (n,):
        raise ValueError("operand shapes do not agree")
    tile_m, tile_n = {"wide": (256, 128), "full": (256, 256)}.get(home, (TILE, TILE))
    if home == "full" and (k < 256 or m * k >= 2 ** 31 or n * k >= 2 ** 31):
        raise ValueError("the 256 x 256 tile needs k >= 256 and operands below 2^31 elements")
    if m % tile_m or n % tile_n or k % TILE_K or a_bits.dtype != np.uint16 or bt_bits.dtype != np.uint16:
        raise ValueError(f"m must be a multiple of {tile_m}, n of {tile_n}, k of 64, operands uint16 bf16 bit patterns")
    buffers = {"a": a_bits, "bt": bt_bits, "bias": bias.astype(np.float32), "scale": scale.astype(np.float32),
               "c": ((m, n), np.uint16), "status": ((1,), np.uint32)}
    return open_hostless(link_json, buffers=buffers, params=lambda addr: params_blobs(addr, m, n, k, home),
                         grid=((m // tile_m) * (n // tile_n),), backend=backend, image=image)
