"""Params blobs of the flash-attention example, packed from buffer addresses (no package imports: the
file can be handed to ``pipec launch --params``)."""
import math
import struct


def params_blobs(addr: dict[str, int], batch: int, q_heads: int, kv_heads: int, seq: int, scale: float | None = None,
                 window: int | None = None) -> dict[str, bytes]:
    """FaCoreParams (56 B) and FaMaskParams (8 B) of include/fa_abi.h; scale defaults to 1 / sqrt(128).  With a window
    the mask blob is addressed to fa.mask.window, else to fa.mask.causal."""
    scale = 1.0 / math.sqrt(128.0) if scale is None else scale
    return {
        "fa.core": struct.pack("<QQQQiiiifi", addr["q"], addr["k"], addr["v"], addr["o"], batch, q_heads, kv_heads, seq,
                               scale * math.log2(math.e), 0),
        ("fa.mask.causal" if window is None else "fa.mask.window"): struct.pack("<ii", seq, window or 0),
    }
