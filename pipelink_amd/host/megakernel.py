"""Host side of the decode megakernel example on the host-less route: one launch = one decoded token."""
from __future__ import annotations

import json
from pathlib import Path

import numpy as np

from ..pipec.launcher import HostlessSession, open_hostless
from ..stages.megakernel import params as mk


def open_session(link_json: str | Path, weights: np.ndarray, kv_cache: np.ndarray, x: np.ndarray, *, layers: int, d: int, hq: int,
                 hkv: int, dff: int, vocab: int, pos: int, workgroups: int, backend=None, image: str | Path | None = None) -> HostlessSession:
    """weights: packed bf16 bit patterns (uint16, see mk_abi.h); kv_cache [L, 2, smax, hkv, 64] uint16 with positions
    0 .. pos-1 filled; x [d] float32.  `workgroups` must be a multiple of hq (each workgroup takes one
    (head, context chunk) of the attention) and no more than can be resident at once: the grid barrier needs every
    workgroup running, so a count above compute units x the link's workgroups per CU is refused.  After a launch and a
    synchronize, `raise_on_status(session)` tells whether the step's barriers all completed."""
    smax = kv_cache.shape[2]
    if kv_cache.shape != (layers, 2, smax, hkv, mk.HEAD_DIM) or kv_cache.dtype != np.uint16 or weights.dtype != np.uint16:
        raise ValueError("kv_cache is [L, 2, smax, hkv, 64] uint16, weights uint16")
    if weights.size != layers * mk.layer_elems(d, hq, hkv, dff) + d + vocab * d:
        raise ValueError("weights do not have the packed size for these dimensions")
    if d % 512 or dff % 512 or (hq * mk.HEAD_DIM) % 512 or hq % hkv or workgroups % hq or pos >= smax or d + 64 > 8192 or dff > 8192:
        raise ValueError("d, dff and hq*64 must be multiples of 512 (dff <= 8192), hq a multiple of hkv, workgroups a multiple of hq, pos < smax")
    if dff % (4 * workgroups):
        raise ValueError("dff must be a multiple of 4 * workgroups")
    chunks = workgroups // hq
    if hq * mk.HEAD_DIM + 3 * workgroups > 8192 + 256:
        raise ValueError("the attention output and the chunk weights do not fit the workgroup's LDS vector")
    if (pos + chunks - 1) // chunks + 1 > 8192 + 256 - 1280:  # the scores sit 1280 floats into the vector
        raise ValueError("a context chunk does not fit the workgroup's LDS vector: use more workgroups")
    link = json.loads(Path(link_json).read_text()) if not isinstance(link_json, dict) else link_json
    prog = mk.program(layers, mk.opcodes_of(link))   # the instruction stream speaks the numbers this link bound
    buffers = {"weights": weights, "kv_cache": kv_cache, "x": x.astype(np.float32), "rope": mk.rope_table(pos), "program": prog,
               "qkv": (((hq + 2 * hkv) * mk.HEAD_DIM,), np.float32), "attn_partial": ((hq * chunks * mk.PARTIAL_STRIDE,), np.float32),
               "h": ((dff,), np.float32), "logits": ((vocab,), np.float32), "sync": ((1024,), np.uint32)}
    blob = lambda addr: {"mk.interp": mk.params_blob(addr, num_instr=len(prog), layers=layers, d=d, hq=hq, hkv=hkv, dff=dff,
                                                     vocab=vocab, pos=pos, smax=smax, chunks=chunks)}
    sess = open_hostless(link_json, buffers=buffers, params=blob, grid=(workgroups,), backend=backend, image=image)
    cus = getattr(sess.backend, "observations", {}).get("observed_cu_count")
    resident = cus * int(sess.link.get("workgroups_per_cu", 1)) if cus else None
    if resident is not None and workgroups > resident:
        sess.close()
        raise ValueError(f"{workgroups} workgroups cannot all be resident on this device ({resident} at most): the grid barrier would never complete")
    return sess


NUM_XCD = 8
STATUS_GAVE_UP = 1


def raise_on_status(sess: HostlessSession) -> np.ndarray:
    """Call after `synchronize()`.  Reads the launch's synchronisation words and raises RuntimeError if a barrier wait
    gave up (status bit 0: the step's outputs are void; x was overwritten, the cache row at `pos` too), if a workgroup
    has not finished, or if the workgroups that share a per-XCD counter (blockIdx % 8) did not all run on one XCC, or
    two such groups ran on the same one (as recorded by the session's first launch) -- the barrier's first level counts on that.  The status word is cleared, so
    the session can be launched again.  Returns the words as read."""
    sync = sess.read("sync")
    problems = []
    status = int(sync[1])
    if status & STATUS_GAVE_UP:
        problems.append("a grid barrier wait gave up")
    if status & ~STATUS_GAVE_UP:
        problems.append(f"unknown status bits {status:#x}")
    if sync[2] != 0:
        problems.append(f"{int(sync[2])} workgroups finished without the last one closing the launch")
    if sync[3] != 0:  # at least one launch has closed: its workgroups recorded where they ran
        ran_on = sync[512:512 + min(512, sess.grid[0])]
        groups = [sorted({int(w) for w in ran_on[x::NUM_XCD]}) for x in range(min(NUM_XCD, sess.grid[0]))]
        if any(len(g) != 1 or not g[0] & 0x100 for g in groups) or len({g[0] for g in groups}) != len(groups):
            problems.append(f"workgroups are not dealt to the XCDs round-robin (recorded XCC words per blockIdx % 8: {groups})")
    if sync[1] != 0:
        cleared = sync.copy()
        cleared[1] = 0
        sess.write("sync", cleared)
    if problems:
        raise RuntimeError("decode megakernel: " + "; ".join(problems))
    return sync
