"""Pack and link the routed-FFN cell on the CPU (hipcc cross-compiles, nothing is launched):
what link.json records, ring depth chosen at link time, rejected mutations of the real cell
(the reference's P3 corpus, campaigns/mok/port/p3/run_p3.py:260-340), the CLI's failure
format, and the host-less launcher's params checks against an in-memory backend."""
import json
import shutil
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest

from pipelink_amd.pipec import linker, plink
from pipelink_amd.pipec.clauses import LaunchError, LinkError, PipeLinkError, SolveError
from pipelink_amd.pipec.launcher import open_hostless
from pipelink_amd.stages.mok import build as mok_build

ROOT = Path(__file__).resolve().parents[1]
pytestmark = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                                reason="needs the ROCm toolchain")


@pytest.fixture(scope="module")
def cell(tmp_path_factory):
    out = tmp_path_factory.mktemp("mokcell")
    res = mok_build.build(out=out, one_unit=False)
    return out, res


def test_link_json_records_the_solved_cell(cell):
    out, res = cell
    link = json.loads((out / "link" / "link.json").read_text())
    assert link["kernel_symbol"] == "pipelink_kernel" and link["threads"] == 256
    # four 16 KB weight buffers, five 16 KB routed-row buffers, 12 KB of scale buffers, the staged task's 1280 bytes + the schedule table fit 160 KB of LDS: the preferred depth is taken
    assert link["bindings"]["pipelink_mok_gemm_depth"] == [4, "solved"]
    # head (4 buffers + 12 KB of scale buffers + the staged task's row tokens and counter copy, whole kernel)
    # + arena (5 buffers, GEMM phase) + schedule table (two prefix-sum tables of 257 entries + the "last workgroup" flag)
    assert link["dyn_smem_bytes"] == (4 * 16384 + 12288 + 1024 + 256) + 5 * 16384 + (2 * 257 * 4 + 8) <= 160 * 1024
    assert link["bindings"]["pipelink_mok_act_arena"][0] == link["bindings"]["pipelink_mok_gemm_arena"][0]  # phase-exclusive
    assert [e["stage_id"] for e in link["params"]["entries"]] == ["mok.framework", "mok.gemm", "mok.act"]
    assert link["params"]["total_bytes"] == 32 + 264 + 40
    assert {e["channel"] for e in link["protocol_expansions"]} == {"gemm_init", "gemm_fini", "gemm_stage", "gemm_ready", "gemm_wait", "gemm_prefetch",
                                                                   "gemm_fwd", "gemm_store", "act_init", "act_fwd",
                                                                   # tiles of few rows / few columns: their own exports
                                                                   "gemm_placement", "gemm_fwd_small", "gemm_store_small", "act_fwd_small"}
    obs = link["observed"]
    assert obs["calls"] == 0 and obs["private_segment_fixed_size"] <= 64 and obs["mfma"] >= 16   # a few dwords spilled in the tile set-up at most
    assert obs["vgpr_count"] <= link["regs_cap"] == 512
    assert link["facts"]["mok.gemm.TILE_X"] == 256
    assert set(link["input_hashes"]) == {"mok.framework", "mok.gemm", "mok.act"}


def _mutated(cell_dir: Path, tmp_path: Path, stage_id: str | None, mutate, pipeline_mutate=None) -> Path:
    """Copy the cell, rewrite one manifest (payload digest recomputed by pack) and/or the pipeline."""
    for f in cell_dir.glob("*.plink"):
        shutil.copy(f, tmp_path / f.name)
    pipeline = json.loads((cell_dir / "pipeline.json").read_text())
    if pipeline_mutate:
        pipeline_mutate(pipeline["pipeline"])
    (tmp_path / "pipeline.json").write_text(json.dumps(pipeline))
    if stage_id:
        manifest, payload = plink.read(tmp_path / f"{stage_id}.plink")
        mutate(manifest)
        manifest["payload"] = {"file": "stage.o"}
        plink.pack(manifest, payload, tmp_path / f"{stage_id}.plink")
    return tmp_path / "pipeline.json"


def test_forced_depth_beyond_lds_is_l_overlap(cell, tmp_path):
    p = _mutated(cell[0], tmp_path, None, None, lambda pl: (pl["handles"]["pipelink_mok_gemm_depth"]["values"].insert(0, 6),
                                                       pl["forced_bindings"].update(pipelink_mok_gemm_depth=6)))
    with pytest.raises(SolveError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert err.value.clause_ids == {"L-OVERLAP"}


def test_act_restricted_to_unclamped_while_cell_forces_clamp_is_l_handle(cell, tmp_path):
    def only_unclamped(m):
        m["stage"]["variants"] = [v for v in m["stage"]["variants"] if v["key"]["pipelink_mok_clamp"] == 0]
    p = _mutated(cell[0], tmp_path, "mok.act", only_unclamped)
    with pytest.raises(SolveError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert err.value.clause_ids == {"L-HANDLE"}


def test_producer_pruned_of_an_export_is_rejected(cell, tmp_path):
    def drop(m):
        del m["stage"]["exports"]["mok_gemm_fwd"]
    p = _mutated(cell[0], tmp_path, "mok.gemm", drop)
    with pytest.raises(PipeLinkError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert err.value.clause_ids == {"L-PROTO"} and "does not declare the export" in str(err.value)


def test_changed_call_declaration_is_l_proto(cell, tmp_path):
    def widen(m):
        for ep in m["endpoints"]:
            if ep["name"] == "act_fwd":
                ep["protocol"]["decl"] = ep["protocol"]["decl"].replace("const MokActTask* task", "const void* task")
                from pipelink_amd.pipec.channels import declaration_digest
                ep["protocol"]["decl_sha256"] = declaration_digest(ep["protocol"]["decl"])
    p = _mutated(cell[0], tmp_path, "mok.framework", widen)
    with pytest.raises(SolveError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert err.value.clause_ids == {"L-PROTO"} and "channels.act_fwd" in str(err.value)


def test_non_persistent_owner_in_persistent_cell_is_l_topo(cell, tmp_path):
    p = _mutated(cell[0], tmp_path, "mok.act", lambda m: m["topology"].update(persistent=False))
    with pytest.raises(LinkError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert err.value.clause_ids == {"L-TOPO"}


def test_stale_shared_declarations_are_refused(cell, tmp_path):
    """An owner repacked against a changed task record must not link with packages built against the
    old one (the hazard the reference's rdc_contrast arm demonstrates, run_p3.py:343-495)."""
    def skew(m):
        for pre in m["hints"]["preludes"]:
            if pre["name"] == "mok_abi.h":
                pre["text"] = pre["text"].replace("int32_t task_idx;", "int32_t task_idx, extra;")
                pre["sha256"] = plink.sha256_hex(pre["text"].encode())
    p = _mutated(cell[0], tmp_path, "mok.act", skew)
    with pytest.raises(LinkError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert "different versions of a shared declaration header" in str(err.value)


def test_cli_prints_named_failures_and_exits_1(cell, tmp_path):
    p = _mutated(cell[0], tmp_path, None, None, lambda pl: pl["exclusive"].append(["instr_gemm", "missing"]))
    proc = subprocess.run([sys.executable, "-m", "pipelink_amd.pipec", "link", str(p), "--out-dir", str(tmp_path / "o"),
                           "--plan-only"], capture_output=True, text=True, cwd=ROOT)
    assert proc.returncode == 1
    assert proc.stderr.strip() == "pipec: [L-PHASE] $.pipeline.exclusive[1][1]: unknown phase"
    ok = subprocess.run([sys.executable, "-m", "pipelink_amd.pipec", "clauses", "--json"], capture_output=True, text=True, cwd=ROOT)
    assert ok.returncode == 0 and {"L-PROTO", "L-HANDLE", "L-PHASE"} <= {r["id"] for r in json.loads(ok.stdout)}
    ins = subprocess.run([sys.executable, "-m", "pipelink_amd.pipec", "inspect", str(cell[0] / "mok.gemm.plink")],
                         capture_output=True, text=True, cwd=ROOT)
    assert ins.returncode == 0 and json.loads(ins.stdout)["stage"]["id"] == "mok.gemm"


class MemoryBackend:
    """Host-memory stand-in for the HIP backend (the reference tests its broker the same way,
    pipec/tests/test_host_broker.py:251-312)."""

    def __init__(self):
        self.mem, self.next, self.launches, self.log = {}, 0x1000, [], []

    def current(self): self.log.append("current")
    def allocate(self, size, align=256):
        addr = self.next
        self.next += (size + 255) // 256 * 256
        self.mem[addr] = bytearray(size)
        self.log.append("allocate")
        return addr
    def free(self, addr): del self.mem[addr]
    def zero(self, addr, size, stream=None): self.mem[addr][:size] = bytes(size)
    def upload(self, addr, data, stream=None):
        self.mem[addr][:len(data)] = data
        self.log.append("upload")
    def readback(self, addr, size, stream=None): return bytes(self.mem[addr][:size])
    def synchronize(self, stream=None): pass
    def module_load(self, image): return 1
    def module_unload(self, module): pass
    def module_function(self, module, name, lds=0): return 2
    def launch(self, fn, params_addr, grid, block, lds, stream=None): self.launches.append((params_addr, grid, block, lds))


def test_hostless_launcher_params_contract(cell):
    link = json.loads((cell[0] / "link" / "link.json").read_text())
    image = cell[0] / "link" / "pipeline.hsaco"
    with pytest.raises(LaunchError) as err:      # a link whose stages declared owners is opened through its providers
        open_hostless(link, buffers={}, params=lambda a: {}, grid=(1,), backend=MemoryBackend(), image=image)
    assert err.value.failures[0].path == "launch.host"
    assert [g["owner"] for g in link.pop("host")["groups"]] == ["mok.framework", "mok.gemm", "mok.act"]
    be = MemoryBackend()
    seen = {}

    def params(addr):
        seen.update(addr)
        assert be.log.count("upload") == 1      # every buffer is in place before params() runs
        return {"mok.framework": b"\x01" * 32, "mok.gemm": b"\x02" * 264, "mok.act": b"\x03" * 40}
    s = open_hostless(link, buffers={"a": np.arange(4, dtype=np.int32), "b": ((8,), np.float32)}, params=params,
                      grid=(16,), backend=be, image=image)
    blob = be.mem[s.params_addr]
    assert blob[0:32] == b"\x01" * 32 and blob[32:296] == b"\x02" * 264 and blob[296:336] == b"\x03" * 40
    s.launch()
    assert be.launches == [(s.params_addr, (16, 1, 1), (256, 1, 1), link["dyn_smem_bytes"])]
    assert s.read("a").tolist() == [0, 1, 2, 3] and s.read("b").tolist() == [0.0] * 8
    s.write("b", np.ones(8, np.float32))
    assert s.read("b").sum() == 8
    other = s.with_image(image)
    other.launch()
    assert len(be.launches) == 2 and be.launches[1][0] == s.params_addr   # shared params and buffers
    s.close()
    refused = MemoryBackend()
    with pytest.raises(LaunchError) as err:
        open_hostless(link, buffers={"a": np.arange(4, dtype=np.int32)}, params=lambda a: {"mok.gemm": b"\0" * 264}, grid=(1,),
                      backend=refused, image=image)
    assert err.value.clause_ids == {"L-PARAMS"} and err.value.failures[0].path == "launch.params"
    assert refused.log.count("allocate") == 1 and not refused.mem       # a refused open gives its device memory back
    with pytest.raises(LaunchError):
        open_hostless(link, buffers={}, params=lambda a: {"mok.framework": b"", "mok.gemm": b"", "mok.act": b""}, grid=(1,),
                      backend=MemoryBackend(), image=image)
