"""Params blob, instruction stream and weight packing of the decode megakernel (no package imports)."""
import math
import struct

import numpy as np

OP_RMSNORM_ATTN, OP_QKV, OP_ATTN, OP_OPROJ, OP_RMSNORM_FFN, OP_UPGATE, OP_DOWN, OP_RMSNORM_FINAL, OP_LMHEAD = range(1, 10)
HEAD_DIM = 64
PARTIAL_STRIDE = HEAD_DIM + 4  # MK_PARTIAL_STRIDE


OPS = ("rmsnorm_attn", "qkv", "attn", "oproj", "rmsnorm_ffn", "upgate", "down", "rmsnorm_final", "lmhead")
DEFAULT_OPCODES = dict(zip(OPS, range(1, 10)))


def opcodes_of(link: dict) -> dict[str, int]:
    """op name -> the number the link bound to its claim (link.json "bindings": pipelink_mk_opcode_<op>)."""
    return {op: link["bindings"][f"pipelink_mk_opcode_{op}"][0] for op in OPS}


def program(layers: int, opcodes: dict[str, int] | None = None) -> np.ndarray:
    """[n, 4] int32 (opcode, layer, barrier_after, 0): the whole decoding step, in the opcode numbers of one link."""
    n = opcodes or DEFAULT_OPCODES
    rows = []
    for l in range(layers):
        rows += [(n["rmsnorm_attn"], l, 0), (n["qkv"], l, 1), (n["attn"], l, 1), (n["oproj"], l, 1),
                 (n["rmsnorm_ffn"], l, 0), (n["upgate"], l, 1), (n["down"], l, 1)]
    rows += [(n["rmsnorm_final"], 0, 0), (n["lmhead"], 0, 0)]
    return np.array([(o, l, b, 0) for o, l, b in rows], dtype=np.int32)


def layer_elems(d: int, hq: int, hkv: int, dff: int) -> int:
    qkv = (hq + 2 * hkv) * HEAD_DIM
    return d + qkv * d + d * hq * HEAD_DIM + d + 2 * dff * d + d * dff


def rope_table(pos: int, theta: float = 500000.0) -> np.ndarray:
    """[2, 32] float32: cos and sin of pos * theta^(-2 i / 64)."""
    inv = theta ** (-np.arange(0, HEAD_DIM, 2, dtype=np.float64) / HEAD_DIM)
    ang = pos * inv
    return np.stack([np.cos(ang), np.sin(ang)]).astype(np.float32)


def params_blob(addr: dict[str, int], *, num_instr: int, layers: int, d: int, hq: int, hkv: int, dff: int, vocab: int, pos: int,
                smax: int, chunks: int, eps: float = 1e-5) -> bytes:
    """MkModel (128 B) of include/mk_abi.h."""
    scale_log2e = (1.0 / math.sqrt(HEAD_DIM)) * math.log2(math.e)
    return struct.pack("<10Q10i2f", addr["weights"], addr["kv_cache"], addr["x"], addr["qkv"], addr["attn_partial"], addr["h"],
                       addr["logits"], addr["rope"], addr["program"], addr["sync"], num_instr, layers, d, hq, hkv, dff, vocab, pos,
                       smax, chunks, eps, scale_log2e)
