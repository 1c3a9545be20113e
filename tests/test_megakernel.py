"""Decode megakernel: an interpreter package and eight op packages linked into one persistent kernel that runs
a whole decoding step; swapping only the attention package and relinking.

CPU part: the oracle's pins, the instruction stream, what the two links record.  GPU part (marked gpu): a small
model against the oracle (logits, residual stream, the appended cache rows), linked vs one-unit byte-identical,
the swapped attention within tolerance of the first; then the stated model (16 layers, d 2048, 32 / 8 heads of 64,
d_ff 8192, vocabulary 128256, 4096 cached positions) against the oracle, with its time per token."""
import json
import shutil
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import llama_decode as ld
from pipelink_amd.stages.megakernel import build as mk_build
from pipelink_amd.stages.megakernel import params as mkp

ROOT = Path(__file__).resolve().parents[1]
needs_rocm = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                                reason="needs the ROCm toolchain")
SMALL = dict(layers=2, d=512, hq=8, hkv=2, dff=1024, vocab=1000, pos=37)


def test_oracle_pieces_against_library_routines_and_invariants():
    g = torch.Generator().manual_seed(0)
    x, w = torch.randn(512, generator=g), (1 + 0.02 * torch.randn(512, generator=g)).to(torch.bfloat16)
    assert torch.allclose(ld.rms_norm(x, w, 1e-5), torch.nn.functional.rms_norm(x, (512,), w.float(), 1e-5), rtol=1e-5, atol=1e-6)
    assert torch.allclose(ld.silu(x), torch.nn.functional.silu(x), rtol=1e-5, atol=1e-6)
    q, k = torch.randn(64, generator=g), torch.randn(64, generator=g)
    assert torch.allclose(ld.rope(q, 123).norm(), q.norm(), rtol=1e-5)                    # a rotation
    assert torch.allclose(ld.rope(q, 0), q)
    a = ld.rope(q, 100) @ ld.rope(k, 90)
    b = ld.rope(q, 40) @ ld.rope(k, 30)
    assert torch.allclose(a, b, rtol=1e-4, atol=1e-4)                                      # depends on the distance only
    assert np.allclose(mkp.rope_table(123)[0], np.cos(123 * 500000.0 ** (-np.arange(0, 64, 2) / 64)), atol=1e-6)


def test_oracle_attention_against_the_library():
    cfg = dict(SMALL, smax=64)
    weights, cache, x = ld.make_model(**cfg, seed=1)
    logits, x2 = ld.decode_step(weights, cache.clone(), x, **SMALL)
    assert torch.isfinite(logits).all() and logits.shape == (1000,) and not torch.equal(x2, x)
    # one head of layer 0 by hand through scaled_dot_product_attention
    w = ld.layer_views(weights, 0, 512, 8, 2, 1024)
    qkv = w["wqkv"].float() @ ld.rms_norm(x, w["attn_norm"], 1e-5)
    q = ld.rope(qkv[:512].view(8, 64), 37)
    c = cache.clone()
    ld.decode_step(weights, c, x, **SMALL)
    keys, vals = c[0, 0, :38, 1].float(), c[0, 1, :38, 1].float()     # KV head 1 serves query heads 4..7
    lib = torch.nn.functional.scaled_dot_product_attention(q[5][None, None], keys[None], vals[None])[0, 0]
    mine = torch.softmax((keys @ q[5]) / 8.0, 0) @ vals
    assert torch.allclose(lib, mine, rtol=1e-5, atol=1e-6)
    assert weights.numel() == 2 * mkp.layer_elems(512, 8, 2, 1024) + 512 + 1000 * 512


def test_program_is_the_whole_step():
    p = mkp.program(16)
    assert p.shape == (16 * 7 + 2, 4) and p.dtype == np.int32
    assert p[:, 2].sum() == 16 * 5                       # five grid barriers per layer
    assert list(p[:7, 0]) == [1, 2, 3, 4, 5, 6, 7] and list(p[-2:, 0]) == [8, 9] and p[-1, 2] == 0
    assert len(mkp.params_blob({k: 0 for k in ("weights", "kv_cache", "x", "qkv", "attn_partial", "h", "logits", "rope", "program", "sync")},
                               num_instr=3, layers=1, d=512, hq=8, hkv=2, dff=1024, vocab=10, pos=1, smax=4, chunks=1)) == 128


@pytest.fixture(scope="module")
def example(tmp_path_factory):
    out = tmp_path_factory.mktemp("megakernel")
    return out, mk_build.build(out=out, one_unit=False)


@needs_rocm
def test_links_nine_packages_and_swaps_only_the_attention(example):
    out, res = example
    link, swap = res["link"], res["swap"]
    assert link["params"]["entries"] == [{"stage_id": "mk.interp", "offset": 0, "bytes": 128, "align": 8}]
    assert link["threads"] == 256 and link["dyn_smem_bytes"] == 33792
    ops = ("qkv", "attn", "oproj", "upgate", "down", "lmhead")
    # the interpreter calls every op; every op but the normalisation calls back once for its inputs (the open half of
    # the grid barrier and the normalisation that is due): one channel per caller
    assert {e["channel"] for e in link["protocol_expansions"]} == {"op_rmsnorm", "rope_apply"} | {f"op_{o}" for o in ops} | {f"inputs_{o}" for o in ops}
    assert link["observed"]["calls"] == 0 and swap["observed"]["calls"] == 0
    same = set(link["input_hashes"]) & set(swap["input_hashes"])
    assert same == {"mk.interp", "mk.rmsnorm", "mk.qkv", "mk.rope", "mk.oproj", "mk.upgate", "mk.down", "mk.lmhead"}
    assert all(link["input_hashes"][s] == swap["input_hashes"][s] for s in same)            # eight packages untouched
    assert "mk.attn" in link["input_hashes"] and "mk.attn.wide" in swap["input_hashes"]


@needs_rocm
def test_opcodes_are_bound_at_link_time(example):
    """The op packages claim slots of the link's opcode domain; the pipeline binds the numbers; a relink with other
    numbers reuses every package (campaigns/megakernel/port/pipelines/{a,rebind-opcode}.json in the reference)."""
    out, res = example
    link, rebind = res["link"], res["rebind"]
    assert mkp.opcodes_of(link) == mkp.DEFAULT_OPCODES
    assert all(link["bindings"][f"pipelink_mk_opcode_{op}"][1] == "forced" for op in mkp.OPS)
    other = mkp.opcodes_of(rebind)
    assert sorted(other.values()) != sorted(mkp.DEFAULT_OPCODES.values()) and len(set(other.values())) == 9
    assert rebind["input_hashes"] == link["input_hashes"]                       # not one package was repacked
    assert [iv["handle"] for iv in link["intervals"]["opcode"]] == [f"pipelink_mk_opcode_{op}" for op in mkp.OPS]
    assert list(mkp.program(1, other)[:3, 0]) == [other["rmsnorm_attn"], other["qkv"], other["attn"]]
    # two ops bound to one number: the claims overlap
    from pipelink_amd.pipec import linker
    from pipelink_amd.pipec.clauses import PipeLinkError
    clash = json.loads((out / "pipeline.json").read_text())
    clash["pipeline"]["forced_bindings"]["pipelink_mk_opcode_down"] = clash["pipeline"]["forced_bindings"]["pipelink_mk_opcode_qkv"]
    (out / "clash.json").write_text(json.dumps(clash))
    with pytest.raises(PipeLinkError) as err:
        linker.link(out / "clash.json", out / "clash", codegen=False)
    assert "L-OVERLAP" in err.value.clause_ids
    # a number past the domain's capacity
    clash["pipeline"]["forced_bindings"]["pipelink_mk_opcode_down"] = 16
    (out / "clash.json").write_text(json.dumps(clash))
    with pytest.raises(PipeLinkError) as err:
        linker.link(out / "clash.json", out / "clash", codegen=False)
    assert "L-OVERLAP" in err.value.clause_ids


class _HostMemory:
    """Host-memory stand-in for the HIP backend: enough for open_session and raise_on_status."""

    def __init__(self, compute_units):
        self.mem, self.next, self.launches = {}, 0x1000, 0
        self.observations = {"observed_cu_count": compute_units}

    def current(self): pass
    def allocate(self, size, align=256):
        addr, self.next = self.next, self.next + (size + 255) // 256 * 256
        self.mem[addr] = bytearray(size)
        return addr
    def free(self, addr): del self.mem[addr]
    def zero(self, addr, size, stream=None): self.mem[addr][:size] = bytes(size)
    def upload(self, addr, data, stream=None): self.mem[addr][:len(data)] = data
    def readback(self, addr, size, stream=None): return bytes(self.mem[addr][:size])
    def synchronize(self, stream=None): pass
    def module_load(self, image): return 1
    def module_unload(self, module): pass
    def module_function(self, module, name, lds=0): return 2
    def launch(self, fn, params_addr, grid, block, lds, stream=None): self.launches += 1


@needs_rocm
def test_host_refuses_grids_that_cannot_be_resident_and_reads_the_status_words(example):
    """The grid barrier needs every workgroup running: open_session refuses more workgroups than compute units x the
    link's workgroups per CU.  raise_on_status turns the launch's words into an error: a wait that gave up, a launch
    that did not close, XCC records that break the round-robin assumption; it clears the sticky status word."""
    from pipelink_amd.host.megakernel import open_session, raise_on_status

    out, res = example
    cfg = dict(SMALL)
    weights, cache, x = ld.make_model(**cfg, smax=64, seed=2)
    args = (out / "link" / "link.json", weights.view(torch.int16).numpy().view(np.uint16), cache.view(torch.int16).numpy().view(np.uint16), x.numpy())
    image = out / "link" / "pipeline.hsaco"
    with pytest.raises(ValueError, match="resident"):
        open_session(*args, workgroups=32, **cfg, backend=_HostMemory(16), image=image)
    be = _HostMemory(32)
    sess = open_session(*args, workgroups=32, **cfg, backend=be, image=image)
    try:
        good = np.zeros(1024, dtype=np.uint32)
        good[3] = 1                                                 # one launch has closed
        good[512:512 + 32] = [0x100 | ((3 * (b % 8)) % 8) for b in range(32)]   # any permutation of the XCCs will do
        sess.write("sync", good)
        assert np.array_equal(raise_on_status(sess), good)
        gave_up = good.copy()
        gave_up[1] = 1
        sess.write("sync", gave_up)
        with pytest.raises(RuntimeError, match="gave up"):
            raise_on_status(sess)
        assert sess.read("sync")[1] == 0                             # cleared: the session can be launched again
        open_launch = good.copy()
        open_launch[2] = 5
        sess.write("sync", open_launch)
        with pytest.raises(RuntimeError, match="finished"):
            raise_on_status(sess)
        for bad in ((512 + 8, 0x101), (512 + 1, 0x100), (512 + 2, 0)):   # two XCCs in one group, one XCC in two groups, none recorded
            words = good.copy()
            words[bad[0]] = bad[1]
            sess.write("sync", words)
            with pytest.raises(RuntimeError, match="round-robin"):
                raise_on_status(sess)
    finally:
        sess.close()


# ---- GPU ---------------------------------------------------------------------------------------------------

def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def _run(paths_key, cfg, weights, cache, x, workgroups, image_key=None, time_launches=0, program=None):
    from pipelink_amd.host.megakernel import open_session

    paths = mk_build.images()
    sess = open_session(paths[paths_key], _bits(weights), _bits(cache), x.numpy(), workgroups=workgroups, **cfg,
                        image=paths[image_key] if image_key else None)
    try:
        if program is not None:
            sess.write("program", program(sess.read("program")))
        from pipelink_amd.host.megakernel import raise_on_status

        sess.launch()
        sess.synchronize()
        out = {n: sess.read(n) for n in ("logits", "x", "kv_cache")}
        barriers = int(sess.read("program")[:, 2].sum())
        _check_sync(raise_on_status(sess), workgroups, barriers, launches=1)
        if time_launches:
            out["ms"] = sorted(sess.time(time_launches) for _ in range(3))[1]   # median of three timings
            sess.synchronize()
            _check_sync(raise_on_status(sess), workgroups, barriers, launches=1 + 3 * time_launches)
        return out
    finally:
        sess.close()


def _check_sync(sync, workgroups, barriers, launches):
    """Every word of the barrier's state after `launches` launches: a launch leaves its counters at zero (each put back
    at the scope it is used at), counts itself in word 3, and the first one recorded where the workgroups ran."""
    assert barriers > 0
    assert sync[0] == 0 and sync[1] == 0 and sync[2] == 0 and sync[3] == launches
    assert not sync[4:512].any()                                  # the per-XCD arrivals, generations and finished counts
    ran_on = [int(w) for w in sync[512:512 + workgroups]]
    assert all(w & 0x100 for w in ran_on)
    groups = [set(ran_on[x::8]) for x in range(min(8, workgroups))]
    assert all(len(g) == 1 for g in groups) and len(set.union(*groups)) == len(groups), groups   # one XCC each, all different
    assert not sync[512 + workgroups:].any()


def _rel(a, b):
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


@pytest.mark.gpu
def test_small_model_matches_the_oracle_linked_one_unit_and_swapped():
    cfg = dict(SMALL)
    weights, cache, x = ld.make_model(**cfg, smax=64, seed=2)
    ref_cache = cache.clone()
    want_logits, want_x = ld.decode_step(weights, ref_cache, x, **cfg)
    got = _run("link_json", cfg, weights, cache, x, workgroups=32)
    assert _rel(got["x"], want_x.numpy()) <= 2e-3 and _rel(got["logits"], want_logits.numpy()) <= 2e-3
    assert int(np.argmax(got["logits"])) == int(torch.argmax(want_logits))
    new_rows = got["kv_cache"][:, :, 37]                                      # the appended key and value of both layers
    ref_rows = _bits(ref_cache)[:, :, 37]
    assert (new_rows != ref_rows).mean() < 0.02                               # bf16 roundings of fp32 sums in another order
    near = torch.from_numpy(new_rows.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    assert _rel(near, ref_cache[:, :, 37].float().numpy()) <= 1e-2
    assert np.array_equal(got["kv_cache"][:, :, :37], _bits(cache)[:, :, :37])  # the rest of the cache untouched
    control = _run("link_json", cfg, weights, cache, x, workgroups=32, image_key="one_unit")
    assert all(np.array_equal(control[n], got[n]) for n in ("logits", "x", "kv_cache")), "linked and one-unit images differ"
    rebound = _run("rebind_link_json", cfg, weights, cache, x, workgroups=32)   # other opcode numbers, same packages
    assert all(np.array_equal(rebound[n], got[n]) for n in ("logits", "x", "kv_cache")), "rebound opcodes changed the result"
    # The barrier's two halves and the held-back normalisation, off the beaten path: the step's last two instructions
    # (final norm, LM head) replaced by an opcode nobody claimed with a barrier behind it (the interpreter itself has to
    # wait for the barrier the down projection opened) and a normalisation as the very last instruction (held back, and
    # nobody asks for it).  x and the cache must come out as from the whole step, the counters in step (_run checks them).
    def detour(prog):
        prog = prog.copy()
        prog[-2] = (0, 0, 1, 0)
        prog[-1] = prog[-5]                      # rmsnorm_ffn of the last layer (it writes only LDS)
        return prog
    off_path = _run("link_json", cfg, weights, cache, x, workgroups=32, program=detour)
    assert np.array_equal(off_path["x"], got["x"]) and np.array_equal(off_path["kv_cache"], got["kv_cache"])
    swapped = _run("swap_link_json", cfg, weights, cache, x, workgroups=32)
    assert _rel(swapped["logits"], got["logits"]) <= 1e-4 and _rel(swapped["logits"], want_logits.numpy()) <= 2e-3


@pytest.mark.gpu
def test_stated_model_against_the_oracle_and_its_time_per_token():
    cfg = dict(layers=16, d=2048, hq=32, hkv=8, dff=8192, vocab=128256, pos=4096)
    weights, cache, x = ld.make_model(**cfg, smax=4104, seed=0)
    print(f"weights {weights.numel() * 2 / 1e9:.2f} GB, cache {cache.numel() * 2 / 1e6:.0f} MB", flush=True)
    want_logits, want_x = ld.decode_step(weights, cache.clone(), x, **cfg)
    got = _run("link_json", cfg, weights, cache, x, workgroups=256, time_launches=20)
    assert _rel(got["x"], want_x.numpy()) <= 5e-3 and _rel(got["logits"], want_logits.numpy()) <= 5e-3
    assert int(np.argmax(got["logits"])) == int(torch.argmax(want_logits))
    bytes_per_token = weights.numel() * 2 + cache[:, :, :4096].numel() * 2
    print(f"decode step: {got['ms']:.3f} ms per token, {bytes_per_token / got['ms'] / 1e9:.2f} TB/s of {bytes_per_token / 1e9:.2f} GB "
          f"(weights + cache read once), {bytes_per_token / got['ms'] / 1e9 / 8 * 100:.1f} % of 8 TB/s", flush=True)
    control = _run("link_json", cfg, weights, cache, x, workgroups=256, image_key="one_unit", time_launches=20)
    assert all(np.array_equal(control[n], got[n]) for n in ("logits", "x", "kv_cache")), "linked and one-unit images differ"
    ratio = control["ms"] / got["ms"]
    print(f"one-unit control: {control['ms']:.3f} ms per token; linked / one-unit throughput ratio {ratio:.4f}", flush=True)
    # (the reference's seam gate is ratio >= 0.97, campaigns/megakernel/evidence/RESULT.md:7: a timing figure, printed
    # here and not asserted -- a correctness suite must not fail on a noisy box)
    swapped = _run("swap_link_json", cfg, weights, cache, x, workgroups=256, time_launches=20)
    assert _rel(swapped["logits"], got["logits"]) <= 1e-4
    print(f"with mk.attn.wide relinked: {swapped['ms']:.3f} ms per token", flush=True)
