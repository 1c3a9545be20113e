"""The three-package GEMM example, C = GELU(A . B + bias): the plumbing case of the reference
(three .plink packages -- loader, MMA, bias+GELU epilogue -- contracts, ring depth solved at link
time, one deliberately mismatched pair that must be named L-PROTO) and its math.

CPU part: the oracle's pins, what the link records, the rejected pair.  GPU part (marked gpu):
the linked image launched on the host-less route against the torch-CPU fp32 result, linked vs
one-unit byte-identical, ring depth 2 vs 4 byte-identical."""
import json
import math
import shutil
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gemm_gelu as gg
from pipelink_amd.pipec import linker, plink
from pipelink_amd.pipec.clauses import PipeLinkError
from pipelink_amd.stages.gemm_split import build as gs_build

ROOT = Path(__file__).resolve().parents[1]


# ---- oracle pins ------------------------------------------------------------------------------

def test_gelu_closed_forms():
    x = np.array([0.0, 1.0, -1.0, 0.5, -3.0, 12.0, -12.0, 40.0, -40.0])
    g = gg.gelu(x)
    assert g[0] == 0.0
    np.testing.assert_allclose(g - gg.gelu(-x), x, rtol=0, atol=1e-15)          # GELU(x) - GELU(-x) = x
    assert g[5] == pytest.approx(12.0, rel=1e-15) and abs(g[6]) < 1e-30         # -> x, -> 0
    assert g[7] == 40.0 and g[8] == 0.0
    assert g[1] == pytest.approx(0.5 * (1 + math.erf(1 / math.sqrt(2))), rel=1e-15)  # = Phi(1) = 0.8413447...
    assert g[1] == pytest.approx(0.8413447460685429, rel=1e-12)


def test_numpy_restatement_agrees_with_the_library_routines():
    a, b, bias = gg.inputs()
    lib = gg.gemm_bias_gelu_torch(a, b, bias).float().numpy()                    # bf16-rounded
    mine = gg.gemm_bias_gelu(a.float().numpy(), b.float().numpy(), bias.numpy())  # fp32
    mine_bf16 = torch.from_numpy(mine).to(torch.bfloat16).float().numpy()
    # different summation orders: a handful of results land on the other side of a bf16 rounding boundary
    assert (gg.bf16_ulp_distance(lib, mine_bf16) > 1.0).sum() == 0
    assert (lib != mine_bf16).mean() < 2e-2
    assert np.linalg.norm(lib - mine) / np.linalg.norm(mine) < 3e-3


def test_inputs_are_the_stated_distribution():
    a, b, bias = gg.inputs()
    assert a.shape == b.shape == (512, 512) and bias.shape == (512,) and a.dtype == torch.bfloat16
    assert a.float().std().item() == pytest.approx(0.05, rel=0.02) and b.float().std().item() == pytest.approx(0.05, rel=0.02)
    assert bias.std().item() == pytest.approx(0.1, rel=0.1)
    a2, _, _ = gg.inputs()
    assert torch.equal(a, a2)


def test_device_erf_approximation_meets_its_bound():
    x = np.linspace(-6.0, 6.0, 200001)
    exact = np.vectorize(math.erf)(x)
    assert np.abs(gg.erf_as(x) - exact).max() < 6e-7   # 1.5e-7 of the formula + fp32 evaluation
    assert gg.erf_as(np.array([0.0]))[0] == pytest.approx(0.0, abs=1e-7)
    assert np.all(gg.erf_as(-x) == -gg.erf_as(x))


# ---- pack + link on the CPU ----------------------------------------------------------------------

needs_rocm = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                                reason="needs the ROCm toolchain")


@pytest.fixture(scope="module")
def example(tmp_path_factory):
    out = tmp_path_factory.mktemp("gemm_split")
    return out, gs_build.build(out=out, one_unit=False)


@needs_rocm
def test_link_records_three_packages_ring_depth_and_geometry(example):
    out, res = example
    link = json.loads((out / "link" / "link.json").read_text())
    assert [e["stage_id"] for e in link["params"]["entries"]] == ["gs.loader", "gs.mma", "gs.epilogue"]
    assert [(e["offset"], e["bytes"]) for e in link["params"]["entries"]] == [(0, 40), (40, 16), (56, 24)]
    assert link["params"]["total_bytes"] == 80
    assert link["threads"] == (4 + 2) * 64 == 384                       # four matrix waves + two loader waves
    assert link["bindings"]["pipelink_gs_depth"] == [4, "solved"]        # deepest ring that fits 160 KB
    assert link["dyn_smem_bytes"] == 4 * 32768 + 2 * 4 * 16 == 131200   # ring + full/empty counter slots
    assert link["bindings"]["pipelink_gs_warp_load"][0] == 0 and link["bindings"]["pipelink_gs_warp_mma"][0] == 2
    exp = {e["channel"]: e for e in link["protocol_expansions"]}
    assert set(exp) == {"ab_ring", "epilogue"}
    ring = exp["ab_ring"]
    assert (ring["kind"], ring["tx_full"], ring["arrive_full"], ring["arrive_empty"]) == ("mbarrier", 32768, 2, 4)   # one arrival per loader wave, one per matrix wave
    assert ring["init_materializer"] == "dispatch" and ring["depth"] == "pipelink_gs_depth"
    assert exp["epilogue"]["kind"] == "call"
    obs = link["observed"]
    assert obs["calls"] == 0 and obs["mfma"] == 16 and obs["private_segment_fixed_size"] == 0
    dispatch = (out / "link" / "dispatch.hip").read_text()
    assert "zero its full/empty counters" in dispatch and "gs_mma_role_mma" in dispatch and "gs_loader_role_load" in dispatch


@needs_rocm
def test_forced_depth_two_halves_the_ring(example, tmp_path):
    for f in example[0].glob("*.plink"):
        shutil.copy(f, tmp_path / f.name)
    pipeline = json.loads((example[0] / "pipeline.json").read_text())
    pipeline["pipeline"]["forced_bindings"] = {"pipelink_gs_depth": 2}
    (tmp_path / "pipeline.json").write_text(json.dumps(pipeline))
    link = linker.link(tmp_path / "pipeline.json", tmp_path / "link", codegen=False)
    assert link["bindings"]["pipelink_gs_depth"] == [2, "forced"] and link["dyn_smem_bytes"] == 2 * 32768 + 2 * 2 * 16 == 65600
    pipeline["pipeline"]["forced_bindings"] = {"pipelink_gs_depth": 8}
    (tmp_path / "pipeline.json").write_text(json.dumps(pipeline))
    with pytest.raises(PipeLinkError) as err:
        linker.link(tmp_path / "pipeline.json", tmp_path / "link8", codegen=False)
    assert [f.clause_id for f in err.value.failures] == ["L-HANDLE"]   # 8 is not one of the handle's declared values


def _relink_with(example_dir: Path, tmp_path: Path, stage_id: str, mutate) -> Path:
    for f in example_dir.glob("*.plink"):
        shutil.copy(f, tmp_path / f.name)
    shutil.copy(example_dir / "pipeline.json", tmp_path / "pipeline.json")
    manifest, payload = plink.read(tmp_path / f"{stage_id}.plink")
    mutate(manifest)
    manifest["payload"] = {"file": "stage.o"}
    plink.pack(manifest, payload, tmp_path / f"{stage_id}.plink")
    return tmp_path / "pipeline.json"


@needs_rocm
def test_mismatched_pair_is_named_l_proto(example, tmp_path):
    """The matrix package built against a ring whose drain takes one arrival per THREAD cannot be
    linked with a loader that waits for one per WAVE."""
    def per_thread(m):
        ring = next(e for e in m["endpoints"] if e["name"] == "ab_ring")
        ring["protocol"]["empty"]["arrive"]["count"] = "threads(mma)"
    p = _relink_with(example[0], tmp_path, "gs.mma", per_thread)
    with pytest.raises(PipeLinkError) as err:
        linker.link(p, tmp_path / "link", codegen=False)
    assert str(err.value) == ("[L-PROTO] channels.ab_ring.protocol.empty.arrive: "
                              "producer and consumer arrival declarations disagree")
    detail = err.value.failures[0].detail
    assert detail["producer"]["count"] == "warps(mma)" and detail["consumer"]["count"] == "threads(mma)"


@needs_rocm
def test_other_mismatches_of_the_pair_are_named_too(example, tmp_path):
    def other_stride(m):
        next(e for e in m["endpoints"] if e["name"] == "ab_ring")["ring"]["stage_stride_bytes"] = 16384
    with pytest.raises(PipeLinkError) as err:
        linker.link(_relink_with(example[0], tmp_path, "gs.mma", other_stride), tmp_path / "l1", codegen=False)
    assert [f.clause_id for f in err.value.failures] == ["L-PROTO"] and "ring" in err.value.failures[0].path

    def other_decl(m):
        call = next(e for e in m["endpoints"] if e["name"] == "epilogue")
        call["protocol"]["decl"] = call["protocol"]["decl"].replace("int wave", "unsigned wave")
    sub = tmp_path / "second"
    sub.mkdir()
    with pytest.raises(PipeLinkError) as err:
        linker.link(_relink_with(example[0], sub, "gs.mma", other_decl), sub / "l2", codegen=False)
    assert "L-PROTO" in [f.clause_id for f in err.value.failures]


@needs_rocm
def test_params_blobs_have_the_packed_sizes(example):
    from pipelink_amd.stages.gemm_split.params import params_blobs

    link = json.loads((example[0] / "link" / "link.json").read_text())
    blobs = params_blobs({"a": 1, "bt": 2, "bias": 3, "c": 4, "status": 5}, 512, 512, 512)
    assert {sid: len(b) for sid, b in blobs.items()} == {e["stage_id"]: e["bytes"] for e in link["params"]["entries"]}


# ---- GPU ----------------------------------------------------------------------------------------------

def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


@pytest.mark.gpu
def test_linked_example_matches_the_cpu_math_and_the_one_unit_control():
    from pipelink_amd.host.gemm_split import open_session

    paths = gs_build.images()
    a, b, bias = gg.inputs()
    want = gg.gemm_bias_gelu_torch(a, b, bias).float().numpy()
    sess = open_session(paths["link_json"], _bits(a), _bits(b.t()), bias.numpy())
    try:
        poison = np.full((512, 512), 0x7FC0, dtype=np.uint16)   # bf16 NaN
        sess.write("c", poison)
        sess.launch()
        sess.synchronize()
        assert sess.read("status")[0] == 0, "a ring wait gave up"
        got_bits = sess.read("c")
        got = torch.from_numpy(got_bits.view(np.int16)).view(torch.bfloat16).float().numpy()
        assert np.isfinite(got).all()
        assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 2e-3     # bf16 output: 2^-9 relative per element at most
        # never more than one bf16 step apart (steps of results below 2^-12 -- sums that cancel -- counted as that of 2^-12)
        assert (gg.bf16_ulp_distance(got, want, floor=2.0 ** -12) > 1.0).sum() == 0
        control = sess.with_image(paths["one_unit"])
        sess.write("c", poison)
        control.launch()
        control.synchronize()
        assert sess.read("status")[0] == 0
        assert np.array_equal(sess.read("c"), got_bits), "linked and one-unit images differ"
        assert sess.time(20) > 0
    finally:
        sess.close()


@pytest.mark.gpu
def test_ring_depth_two_gives_the_same_bytes(tmp_path):
    from pipelink_amd.host.gemm_split import open_session

    paths = gs_build.images()
    shallow = {"link_json": ROOT / "pipelink_amd" / "stages" / "gemm_split" / "build_depth2" / "link" / "link.json"}
    assert shallow["link_json"].exists(), "gemm_split example (depth 2) is not built: run __graft_entry__.build()"
    a, b, bias = gg.inputs(256, 384, 320, seed=5)      # ragged tile counts, five ring stages
    out = []
    for p in (paths, shallow):
        sess = open_session(p["link_json"], _bits(a), _bits(b.t()), bias.numpy())
        try:
            sess.launch()
            sess.synchronize()
            assert sess.read("status")[0] == 0
            out.append(sess.read("c"))
        finally:
            sess.close()
    assert json.loads(shallow["link_json"].read_text())["bindings"]["pipelink_gs_depth"] == [2, "forced"]
    assert np.array_equal(out[0], out[1])
    want = gg.gemm_bias_gelu_torch(a, b, bias).float().numpy()
    got = torch.from_numpy(out[0].view(np.int16)).view(torch.bfloat16).float().numpy()
    assert (gg.bf16_ulp_distance(got, want, floor=2.0 ** -12) > 1.0).sum() == 0


@needs_rocm
def test_launch_verb_checks_its_arguments_before_touching_a_device(example, tmp_path):
    from pipelink_amd.pipec import launcher
    from pipelink_amd.pipec.clauses import LaunchError

    link = example[0] / "link" / "link.json"
    with pytest.raises(LaunchError) as err:
        launcher.launch(link, grid=None)
    assert str(err.value) == "[L-LAUNCH] launch.grid: host-less launch requires a grid"
    with pytest.raises(LaunchError) as err:
        launcher.launch(link, grid=(16,), providers={"gs": "libx.so"})
    assert err.value.failures[0].path == "launch.providers"
    with pytest.raises(LaunchError) as err:
        launcher.launch(link, grid=(16,), params="x.py:f", blobs={"gs.mma": "b.bin"})
    assert "mutually exclusive" in str(err.value)
    with pytest.raises(LaunchError) as err:
        launcher.launch(link, grid=(16,), buffers={"c": "512x512:uint16"}, outputs={"d": str(tmp_path / "d.npy")})
    assert err.value.failures[0].path == "launch.outputs"
    with pytest.raises(LaunchError) as err:
        launcher.launch(link, grid=(16,), buffers={"c": "512by512"})
    assert err.value.failures[0].path == "launch.buffers"
    builder = launcher._load_params_function(str(ROOT / "pipelink_amd" / "stages" / "gemm_split" / "params.py") + ":params_512")
    assert set(builder({"a": 1, "bt": 2, "bias": 3, "c": 4, "status": 5})) == {"gs.loader", "gs.mma", "gs.epilogue"}


@pytest.mark.gpu
def test_cli_launch_verb_runs_the_example(tmp_path):
    import subprocess
    import sys

    paths = gs_build.images()
    a, b, bias = gg.inputs()
    np.save(tmp_path / "a.npy", _bits(a))
    np.save(tmp_path / "bt.npy", _bits(b.t()))
    np.save(tmp_path / "bias.npy", bias.numpy())
    cmd = [sys.executable, "-m", "pipelink_amd.pipec", "launch", str(paths["link_json"]), "--grid", "16",
           "--buffer", f"a={tmp_path / 'a.npy'}", "--buffer", f"bt={tmp_path / 'bt.npy'}", "--buffer", f"bias={tmp_path / 'bias.npy'}",
           "--buffer", "c=512x512:uint16", "--buffer", "status=1:uint32",
           "--params", str(ROOT / "pipelink_amd" / "stages" / "gemm_split" / "params.py") + ":params_512",
           "--output", f"c={tmp_path / 'c.npy'}", "--output", f"status={tmp_path / 'status.npy'}"]
    proc = subprocess.run(cmd, capture_output=True, text=True, cwd=ROOT, timeout=120)
    assert proc.returncode == 0, proc.stderr
    report = json.loads(proc.stdout)
    assert report["geometry"] == {"grid": [16, 1, 1], "block": [384, 1, 1], "dynamic_smem_bytes": 131200}
    assert np.load(tmp_path / "status.npy")[0] == 0
    got = torch.from_numpy(np.load(tmp_path / "c.npy").view(np.int16)).view(torch.bfloat16).float().numpy()
    want = gg.gemm_bias_gelu_torch(a, b, bias).float().numpy()
    assert (gg.bf16_ulp_distance(got, want, floor=2.0 ** -12) > 1.0).sum() == 0
