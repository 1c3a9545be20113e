"""One epilogue, many producers: a bf16 GEMM whose accumulator lives in AGPRs, in VGPRs or in an LDS tile,
and ONE epilogue package (per-column scale + bias, bf16 out) linked against each; the linker generates the
accumulator import for the producer's home.

CPU part: the three links (routes, ring depth, the epilogue package byte for byte the same in all three),
the rejected connections.  GPU part (marked gpu): M = N = K = 8192 -- every linked image byte-identical to
its one-unit control and to the other homes, sampled rows against torch-CPU fp32 within the bf16 bar."""
import json
import shutil
from pathlib import Path

import numpy as np
import pytest
import torch

from oracle import gemm_gelu as gg
from pipelink_amd.pipec import linker, plink
from pipelink_amd.pipec.clauses import PipeLinkError
from pipelink_amd.stages.one_epilogue import build as oe_build

ROOT = Path(__file__).resolve().parents[1]
needs_rocm = pytest.mark.skipif(shutil.which("hipcc") is None and not Path("/opt/rocm/bin/hipcc").exists(),
                                reason="needs the ROCm toolchain")


def test_scale_bias_oracle_pins():
    a, b, scale, bias = gg.scale_bias_inputs(64, 96, 128, seed=3)
    full = gg.gemm_scale_bias_torch(a, b, scale, bias).float()
    acc = a.double() @ b.double()
    want = (acc * scale.double() + bias.double())
    assert (full.double() - want).abs().max() <= want.abs().max() * 2.0 ** -8        # bf16 rounding of the result
    rows = torch.tensor([5, 0, 63])
    assert torch.equal(gg.gemm_scale_bias_torch(a, b, scale, bias, rows).float(), full[rows])
    zero = gg.gemm_scale_bias_torch(a, b, torch.zeros_like(scale), bias).float()
    assert torch.equal(zero, bias.to(torch.bfloat16).float().expand(64, 96))          # scale 0 leaves the bias
    assert a.float().std().item() == pytest.approx(0.02, rel=0.05)


@pytest.fixture(scope="module")
def example(tmp_path_factory):
    out = tmp_path_factory.mktemp("one_epilogue")
    return out, oe_build.build(out=out, one_unit=False)


@needs_rocm
def test_one_epilogue_package_links_against_three_homes(example):
    out, res = example
    links = res["links"]
    routes = {h: links[h]["tensor_plans"][0]["route"] for h in oe_build.HOMES}
    assert routes == {"agpr": "accvgpr_receipt", "vgpr": "register_copy", "lds": "lds_load"}
    # the same epilogue and loader packages, byte for byte, in all three links
    assert len({links[h]["input_hashes"]["oe.epilogue"] for h in oe_build.HOMES}) == 1
    assert len({links[h]["input_hashes"]["gs.loader"] for h in oe_build.HOMES}) == 1
    # registers: the deepest ring fits; the LDS home claims 4 x 64 x 272 B of tiles and the ring settles for depth 2
    assert links["agpr"]["bindings"]["pipelink_gs_depth"] == links["vgpr"]["bindings"]["pipelink_gs_depth"] == [4, "solved"]
    assert links["lds"]["bindings"]["pipelink_gs_depth"] == [2, "solved"]
    assert links["lds"]["dyn_smem_bytes"] == 2 * 32768 + 4 * 64 * 272 + 2 * 2 * 16 == 135232
    assert links["agpr"]["observed"]["agpr_count"] >= 64 and links["vgpr"]["observed"]["agpr_count"] == 0
    for h in oe_build.HOMES:
        assert links[h]["observed"]["calls"] == 0 and links[h]["observed"]["private_segment_fixed_size"] == 0
        stub = (out / h / "link" / "stub.hip").read_text()
        assert "oe_epilogue_import_acc(const void* source, float* dest)" in stub and f"route {routes[h]}" in stub
    assert "v_accvgpr_read_b32" in (out / "agpr" / "link" / "stub.hip").read_text()


def _relink(example_dir: Path, tmp_path: Path, home: str, stage_id: str | None, mutate, pipeline_mutate=None) -> Path:
    for f in (example_dir / home).glob("*.plink"):
        shutil.copy(f, tmp_path / f.name)
    pipeline = json.loads((example_dir / home / "pipeline.json").read_text())
    if pipeline_mutate:
        pipeline_mutate(pipeline["pipeline"])
    (tmp_path / "pipeline.json").write_text(json.dumps(pipeline))
    if stage_id:
        manifest, payload = plink.read(tmp_path / f"{stage_id}.plink")
        mutate(manifest)
        manifest["payload"] = {"file": "stage.o"}
        plink.pack(manifest, payload, tmp_path / f"{stage_id}.plink")
    return tmp_path / "pipeline.json"


@needs_rocm
def test_wide_tile_links_its_own_trio(example):
    """256 x 128 workgroup tiles: three loader waves + four matrix waves, three stages of 48 KB in the ring, the wave's
    128 x 64 accumulator in AGPRs handed to the epilogue one 32 x 32 block at a time."""
    out, res = example
    wide = res["links"]["wide"]
    assert [e["stage_id"] for e in wide["params"]["entries"]] == ["oe.loader.wide", "oe.mma.wide", "oe.epilogue.wide"]
    assert wide["threads"] == 7 * 64 and wide["bindings"]["pipelink_gs_depth"] == [3, "solved"]
    assert wide["dyn_smem_bytes"] == 3 * (256 + 128) * 128 + 2 * 3 * 16 <= 160 * 1024
    plan = wide["tensor_plans"][0]
    assert plan["route"] == "accvgpr_receipt" and plan["function"] == "oe_epilogue_wide_import_acc"
    obs = wide["observed"]
    # two waves share a SIMD (7 waves on 4): 256 registers each at most
    assert obs["calls"] == 0 and obs["private_segment_fixed_size"] == 0 and obs["agpr_count"] == 128 and obs["vgpr_count"] <= 256
    stub = (out / "wide" / "link" / "stub.hip").read_text()
    assert "oe_epilogue_wide_import_acc_block(const void* source, int block, float* dest)" in stub


@needs_rocm
def test_full_tile_links_a_matrix_package_that_loads_its_own_operands(example):
    """256 x 256 workgroup tiles: four waves with 128 x 128 each in all 256 AGPRs and no loader waves beside them, two
    rings of five 16 KB buffers (all of the LDS), the accumulator handed over transposed, block by block."""
    out, res = example
    full = res["links"]["full"]
    assert [e["stage_id"] for e in full["params"]["entries"]] == ["oe.mma.full", "oe.epilogue.full"]
    assert full["threads"] == 4 * 64 and full["dyn_smem_bytes"] == 2 * 5 * 256 * 64 == 160 * 1024
    plan = full["tensor_plans"][0]
    assert plan["route"] == "accvgpr_receipt" and plan["function"] == "oe_epilogue_full_import_acc"
    obs = full["observed"]
    # one wave per SIMD: the whole register file of a lane, nothing spilled; six steps of 32 MFMAs are written out
    assert obs["calls"] == 0 and obs["private_segment_fixed_size"] == 0 and obs["agpr_count"] == 256 and obs["vgpr_spill_count"] == 0
    assert obs["mfma"] == 6 * 32
    stub = (out / "full" / "link" / "stub.hip").read_text()
    assert "oe_epilogue_full_import_acc_block(const void* source, int block, float* dest)" in stub


@needs_rocm
def test_rejected_tensor_connections_are_named(example, tmp_path):
    cases = [
        ("vgpr", "oe.mma.vgpr", lambda m: m["tensor"]["exports"][0].update(dtype="f16"), None, "T-CONTRACT",
         "pipeline.tensor_connections.acc", "exported and imported tensor identities disagree"),
        ("vgpr", "oe.mma.vgpr", lambda m: m["tensor"]["exports"][0].update(home="tmem"), None, "T-PLAN",
         "pipeline.tensor_connections.acc", "no transport route reads this home and layout"),
        ("lds", "oe.mma.lds", lambda m: m["tensor"]["exports"][0].update(row_pitch_bytes=128), None, "T-CONTRACT",
         "pipeline.tensor_connections.acc", "row pitch of the exported tile is smaller than a row or not a multiple of 4"),
        ("agpr", None, None, lambda p: p.update(tensor_connections=[]), "T-CONTRACT",
         "stages.oe.epilogue.tensor.imports.acc", "import is not fed by any tensor connection"),
        ("agpr", None, None, lambda p: p["tensor_connections"][0].update(export="accumulator"), "T-CONTRACT",
         "pipeline.tensor_connections.acc", "connection names an export or import its stage does not declare"),
    ]
    for i, (home, sid, mutate, pmutate, clause, path, message) in enumerate(cases):
        sub = tmp_path / str(i)
        sub.mkdir()
        with pytest.raises(PipeLinkError) as err:
            linker.link(_relink(example[0], sub, home, sid, mutate, pmutate), sub / "link", codegen=False)
        first = err.value.failures[0]
        assert (first.clause_id, first.path, first.message) == (clause, path, message), str(err.value)


# ---- GPU ---------------------------------------------------------------------------------------------------

def _bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def test_host_rejects_shapes_a_tile_does_not_handle():
    """Each cell states its tile: 128 x 128 (the three homes), 256 x 128 (wide), 256 x 256 with a contraction of at
    least 256 (full); anything else is refused before a buffer is allocated."""
    from pipelink_amd.host.one_epilogue import open_session

    z = lambda *shape: np.zeros(shape, dtype=np.uint16)
    f = lambda n: np.zeros(n, dtype=np.float32)
    bad = [("agpr", 192, 128, 64), ("agpr", 128, 128, 96), ("wide", 128, 128, 64), ("wide", 256, 192, 64),
           ("full", 256, 384, 256), ("full", 384, 256, 256), ("full", 256, 256, 128), ("full", 256, 256, 288)]
    for home, m, n, k in bad:
        with pytest.raises(ValueError):
            open_session("unused.json", home, z(m, k), z(n, k), f(n), f(n))
    with pytest.raises(ValueError):
        open_session("unused.json", "full", z(256, 256), z(256, 512), f(256), f(256))   # contractions differ


def _print_sustained(sess, home, flop):
    """Sustained rate of the linked image (printed, not asserted): 100 launches back to back after a 1 s ramp, the
    median of five such runs, with the board's power and clock sampled meanwhile."""
    import time

    import bench

    end = time.perf_counter() + 1.0
    while time.perf_counter() < end:
        sess.time(50)
    with bench.PowerSampler() as power:
        ms = sorted(sess.time(100) for _ in range(5))[2]
    rep = power.report()
    print(f"{home}: sustained {ms:.3f} ms = {flop / ms / 1e9:.0f} TFLOP/s at {rep['draw_w']} W of {rep['cap_w']} W, "
          f"{rep['sclk_mhz']} MHz ({rep['samples']} samples)", flush=True)


@pytest.mark.gpu
@pytest.mark.parametrize("size", [512, (256, 256, 256), (512, 256, 320), (768, 512, 1088), 8192], ids=str)
def test_three_homes_one_epilogue_bit_exact_and_within_the_bf16_bar(size):
    """Square sizes, the shortest contractions the 256 x 256 tile takes (8 and 10 slots of 32 elements: its loop's
    prologue and tail with one or two steady steps between), and one where m, n and k all differ (three row tiles of
    the 256-row tiles, an odd number of ring stages)."""
    from pipelink_amd.host.one_epilogue import open_session

    m, n, k = size if isinstance(size, tuple) else (size, size, size)
    a, b, scale, bias = gg.scale_bias_inputs(m, n, k, seed=0)
    a_bits, bt_bits = _bits(a), _bits(b.t())
    results = {}
    for home in oe_build.CELLS:
        paths = oe_build.images(home)
        sess = open_session(paths["link_json"], home, a_bits, bt_bits, bias.numpy(), scale.numpy())
        try:
            print(f"home {home} m {m} n {n} k {k}", flush=True)
            sess.launch()
            sess.synchronize()
            assert sess.read("status")[0] == 0, "a ring wait gave up"
            results[home] = sess.read("c")
            control = sess.with_image(paths["one_unit"])
            sess.write("c", np.full((m, n), 0x7FC0, dtype=np.uint16))    # bf16 NaN
            control.launch()
            control.synchronize()
            assert sess.read("status")[0] == 0
            assert np.array_equal(sess.read("c"), results[home]), f"{home}: linked and one-unit images differ"
            if m == 8192 and home in ("agpr", "wide", "full"):
                _print_sustained(sess, home, 2.0 * m * n * k)
        finally:
            sess.close()
    assert np.array_equal(results["agpr"], results["vgpr"]) and np.array_equal(results["agpr"], results["lds"])
    # the wide tile multiplies the same 16-element steps in the same order: the same bits
    assert np.array_equal(results["agpr"], results["wide"])
    # so does the 256 x 256 tile, with the operands' roles swapped (it accumulates the transpose)
    assert np.array_equal(results["agpr"], results["full"])
    rows = torch.arange(m) if m <= 768 else torch.from_numpy(np.random.default_rng(0).choice(m, 48, replace=False))
    want = gg.gemm_scale_bias_torch(a, b, scale, bias, rows).float().numpy()
    got = torch.from_numpy(results["agpr"].view(np.int16)).view(torch.bfloat16).float().numpy()[rows.numpy()]
    assert np.isfinite(got).all()
    rel = np.abs(got - want) / np.maximum(np.abs(want), 2.0 ** -6)   # results are O(0.1); a floor for the few near zero
    assert rel.max() <= 1e-2
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= 3e-3
