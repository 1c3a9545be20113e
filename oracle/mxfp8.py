"""MXFP8 number formats and the block quantiser, restated on the CPU in numpy.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).  Bit arithmetic throughout so
that no library cast decides a rounding.

Formats
-------
* e4m3 is OCP "E4M3FN": 1 sign, 4 exponent (bias 7), 3 mantissa bits, no infinities,
  NaN = S.1111.111, largest finite 448, smallest subnormal 2**-9.
* e8m0 is an unsigned power of two: value 2**(b-127), b = 255 is NaN.

Block quantiser (OCP Microscaling v1.0, 32-element blocks along the contraction dim)
-------------------------------------------------------------------------------------
For a block ``v[0..31]``:  ``amax = max|v|``;  ``E = floor(log2(amax))`` taken from the
fp32 exponent field;  scale byte ``b = clamp(E - 8 + 127, 0, 254)`` (8 = emax of e4m3);
``amax == 0`` or subnormal gives ``b = 0``.  Elements are
``e4m3_rne(clamp(v * 2**(127 - b), -448, 448))``.  The operand layout follows
campaigns/mok/port/gemm/provider.cu:70-108 (activations ``[rows, K]``, weights
``[N, K]``, one scale per 1x32 block along K); the scale tensor here is plain row-major
``[rows, K/32]`` padded to a multiple of 4 columns.
"""
from __future__ import annotations

import numpy as np

E4M3_MAX = 448.0
MX_BLOCK = 32


def e4m3_decode_table() -> np.ndarray:
    """All 256 e4m3fn codes as float32, from the format definition."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        sign = -1.0 if code & 0x80 else 1.0
        exp = (code >> 3) & 0xF
        man = code & 0x7
        if exp == 0xF and man == 0x7:
            val = float("nan")
        elif exp == 0:
            val = sign * man * 2.0 ** -9
        else:
            val = sign * (1.0 + man / 8.0) * 2.0 ** (exp - 7)
        out[code] = val
    return out


_DECODE = e4m3_decode_table()


def e4m3_decode(codes: np.ndarray) -> np.ndarray:
    return _DECODE[np.asarray(codes, dtype=np.uint8)]


def e4m3_encode(x: np.ndarray) -> np.ndarray:
    """fp32 -> e4m3fn code, round-to-nearest-even, saturating at +-448, NaN -> 0x7F|sign."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32)
    sign = ((bits >> 24) & 0x80).astype(np.uint8)
    nan = np.isnan(x)
    a = np.minimum(np.abs(np.where(nan, np.float32(0), x)), np.float32(E4M3_MAX)).astype(np.float32)
    ab = a.view(np.uint32).astype(np.uint64)
    # normal range: keep 3 mantissa bits, RNE on the 20 dropped bits
    rounded = (ab + 0x7FFFF + ((ab >> 20) & 1)) >> 20  # = (exp_field << 3) | mantissa
    normal_code = rounded.astype(np.int64) - ((127 - 7) << 3)
    # subnormal range (a < 2**-6): multiples of 2**-9; rint is RNE; result 8 is the first normal
    sub_code = np.rint(a.astype(np.float64) * 512.0).astype(np.int64)
    code = np.where(a < np.float32(2.0 ** -6), sub_code, normal_code)
    code = np.clip(code, 0, 0x7E).astype(np.uint8)
    code = np.where(nan, np.uint8(0x7F), code)
    return (code | sign).astype(np.uint8)


def e8m0_decode(b: np.ndarray) -> np.ndarray:
    """2**(b-127) as float32 (b = 0 gives the fp32 subnormal 2**-127, b = 255 NaN)."""
    b = np.asarray(b, dtype=np.uint8).astype(np.int32)
    out = np.ldexp(np.float64(1.0), b - 127).astype(np.float32)
    return np.where(b == 255, np.float32("nan"), out)


def e8m0_from_amax(amax: np.ndarray) -> np.ndarray:
    """Scale byte for a block whose largest magnitude is ``amax`` (fp32, >= 0)."""
    amax = np.ascontiguousarray(amax, dtype=np.float32)
    efield = ((amax.view(np.uint32) >> 23) & 0xFF).astype(np.int32)  # floor(log2)+127, 0 if subnormal/0
    return np.clip(efield - 8, 0, 254).astype(np.uint8)


def padded_scale_cols(k: int) -> int:
    """Leading dimension of a scale row: K/32 rounded up to a multiple of 4 bytes."""
    return ((k // MX_BLOCK) + 3) // 4 * 4


def mx_quantize(x: np.ndarray) -> tuple[np.ndarray, np.ndarray]:
    """Quantise the last axis in 32-blocks.  Returns (codes u8 [..., K], scales u8 [..., ld])
    with ``ld = padded_scale_cols(K)``; padding bytes are 0."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    k = x.shape[-1]
    assert k % MX_BLOCK == 0, "K must be a multiple of 32"
    nb = k // MX_BLOCK
    blk = x.reshape(x.shape[:-1] + (nb, MX_BLOCK))
    amax = np.max(np.abs(blk), axis=-1)
    b = e8m0_from_amax(amax)
    inv = np.ldexp(np.float64(1.0), 127 - b.astype(np.int32)).astype(np.float32)  # exact power of two
    scaled = (blk * inv[..., None]).astype(np.float32)
    codes = e4m3_encode(scaled).reshape(x.shape)
    sc = np.zeros(x.shape[:-1] + (padded_scale_cols(k),), dtype=np.uint8)
    sc[..., :nb] = b
    return codes, sc


def mx_dequantize(codes: np.ndarray, sc: np.ndarray) -> np.ndarray:
    """Inverse map to float32: e4m3 value times 2**(b-127); exact in fp32 for finite results."""
    k = codes.shape[-1]
    nb = k // MX_BLOCK
    vals = e4m3_decode(codes).reshape(codes.shape[:-1] + (nb, MX_BLOCK))
    scale = e8m0_decode(sc[..., :nb])
    return (vals * scale[..., None]).astype(np.float32).reshape(codes.shape)


def bf16_round(x: np.ndarray) -> np.ndarray:
    """fp32 -> nearest-even bf16 -> fp32, by bit arithmetic (NaN kept quiet)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    bits = x.view(np.uint32).astype(np.uint64)
    r = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    out = (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32)
    return np.where(np.isnan(x), np.float32("nan"), out)


def bf16_bits(x: np.ndarray) -> np.ndarray:
    """fp32 -> bf16 bit patterns (uint16), RNE."""
    return (bf16_round(x).view(np.uint32) >> 16).astype(np.uint16)
