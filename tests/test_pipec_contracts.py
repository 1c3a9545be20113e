"""Contract checking of pipec on CPU: the reference's negative fixtures (named clause + path),
the six contract-gallery diagnostics with their verbatim wording, ring-depth known answers and
solver determinism."""
import copy
import glob
import itertools
import json
import os

import pytest

from pipelink_amd.pipec import channels, glue, linker, manifest, solver
from pipelink_amd.pipec.clauses import CLAUSES, ClauseFailure, LinkError, PipeLinkError, SchemaError, SolveError, register_clause

HERE = os.path.dirname(os.path.abspath(__file__))
ZERO = "0" * 64


def abi(profile="sm_103a"):
    return {"schema": "3.0", "target": {"profile": profile, "lto_arch": "lto", "toolkit": "test"}}


def stage(stage_id, roles, *, endpoints=None, claims=None, exports=None, variants=None, profile="sm_103a",
          params=(16, 16), persistent=False):
    prefix = stage_id.replace(".", "_").replace("-", "_") + "_"
    return {"pipelink_abi": abi(profile),
            "stage": {"id": stage_id, "version": "1.0.0", "symbol_prefix": prefix, "entry_abi": "v2",
                      "roles": {r: {"entry": f"{prefix}role_{r}", "warps": w} for r, w in roles.items()},
                      "exports": exports or {}, "entry_signature": "void(const void* params, unsigned variant)",
                      "variants": variants or [{"key": {}, "index": 0}]},
            "endpoints": endpoints or [], "claims": claims or [],
            "topology": {"cta_group": {"fixed": 1}, "cluster": {"compiled": [1, 1, 1], "launch": {"x_multiple_of": 1, "max": [4, 4, 1]}},
                         "multicast": [], "persistent": persistent, "scheduler": "static"},
            "params": {"bytes": params[0], "align": params[1], "type": f"{prefix}Params", "sha256_of_layout_probe": ZERO}}


def pipeline(stage_ids, handles, *, phases=None, profile="sm_103a", persistent=False, forced=None):
    return {"pipelink_abi": abi(profile),
            "pipeline": {"name": "fixture", "stages": [{"artifact_path": f"{s}.plink", "stage_id": s} for s in stage_ids],
                         "handles": handles, "phases": phases or ["steady"], "exclusive": [],
                         "domains": {"gmem_counter": {"capacity": 16}},
                         "depth_priority": [n for n, h in handles.items() if h["class"] == "depth"], "regs_priority": [],
                         "forced_bindings": forced or {}, "topology": {"persistent": persistent, "scheduler": "static"}}}


def ring_endpoint(name, direction, role, full, shape=(4, 4), stride=32):
    return {"name": name, "direction": direction, "owner_role": role, "space": "smem", "scope": "cta", "proxy": "async",
            "tile": {"dtype": "bf16", "shape": list(shape)},
            "layout": {"encoding": "pl-layout-v2", "elem_bits": 16, "shape": [[shape[0]], [shape[1]]], "stride": [[shape[1]], [1]]},
            "ring": {"depth": {"handle": "pipelink_depth"}, "stage_stride_bytes": stride},
            "protocol": {"kind": "mbarrier", "full": copy.deepcopy(full),
                         "empty": {"slots": "pipelink_empty", "arrive": {"count": "threads(mma)", "by": "mma"}, "tx_bytes": 0},
                         "init": {"owner": "load", "materializer": "dispatch", "phase": 0}, "release": "once-per-acquire"},
            "binds": {"full": "pipelink_full", "empty": "pipelink_empty"}}


RING_HANDLES = {"pipelink_depth": {"class": "depth", "binding": "bind", "values": [2, 4], "owner": "channel:ring"},
                "pipelink_empty": {"class": "base", "binding": "bind", "domain": "mbarrier", "owner": "claim:empty"},
                "pipelink_full": {"class": "base", "binding": "bind", "domain": "mbarrier", "owner": "claim:full"}}
RING_CLAIMS = [{"domain": "mbarrier", "handle": h, "extent": {"const": 0, "per": {"pipelink_depth": 1}}, "align": 1}
               for h in ("pipelink_full", "pipelink_empty")]
FULL = {"slots": "pipelink_full", "arrive": {"count": 1, "by": "load"}, "tx_bytes": "tile"}


def barrier_base():
    return {"stages": [stage("alpha.stage", {"load": 4}, endpoints=[ring_endpoint("ring", "produce", "load", FULL)], claims=copy.deepcopy(RING_CLAIMS)),
                       stage("beta.stage", {"mma": 4}, endpoints=[ring_endpoint("ring", "consume", "mma", FULL)])],
            "pipeline": pipeline(["alpha.stage", "beta.stage"], copy.deepcopy(RING_HANDLES))}


def double_barrier_base():
    root = barrier_base()
    root["stages"][0]["endpoints"].append(ring_endpoint("other", "produce", "load", FULL))
    root["stages"][1]["endpoints"].append(ring_endpoint("other", "consume", "mma", FULL))
    return root


def shared_completion_base():
    """Three tile channels whose `full` sides complete on one counter: `root` owns it, `member` and `leaf` name it."""
    names = ("root", "member", "leaf")
    root_full = {"slots": "pipelink_full", "arrive": {"count": 1, "by": "load"}, "tx_bytes": {"sum": list(names)}}
    member_full = {"member_of": "root", "tx_bytes": "tile"}

    def eps(direction, role):
        return [ring_endpoint("root", direction, role, root_full), ring_endpoint("member", direction, role, member_full, shape=(2, 2)),
                ring_endpoint("leaf", direction, role, member_full, shape=(2, 2))]
    return {"stages": [stage("alpha.stage", {"load": 4}, endpoints=eps("produce", "load"), claims=copy.deepcopy(RING_CLAIMS)),
                       stage("beta.stage", {"mma": 4}, endpoints=eps("consume", "mma"))],
            "pipeline": pipeline(["alpha.stage", "beta.stage"], copy.deepcopy(RING_HANDLES))}


def symbols_base():
    """Two artifacts' tables of strong symbols (what `pipec pack` records from each object file)."""
    return {"tables": {"alpha.stage": {"strong": ["alpha_stage_entry"]}, "beta.stage": {"strong": ["beta_stage_entry"]}}}


def call_base():
    decl = 'extern "C" int beta_stage_compute(int value);'
    caller = 'extern "C" int pipelink_call_invoke(int value);'

    def ep(direction):
        d = caller if direction == "produce" else decl
        return {"name": "invoke", "direction": direction, "owner_role": "load" if direction == "produce" else None,
                "space": "reg", "scope": "cta", "proxy": "generic", "tile": {"dtype": "s32", "shape": [128, 1]},
                "layout": {"encoding": "pl-layout-v2", "elem_bits": 32, "shape": [128, 1], "stride": [1, 1]},
                "protocol": {"kind": "call", "export": "compute", "signature": "int(int)", "decl": d,
                             "decl_sha256": channels.declaration_digest(d)}, "binds": {}}
    return {"stages": [stage("alpha.stage", {"load": 4}, endpoints=[ep("produce")]),
                       stage("beta.stage", {"mma": 4}, endpoints=[ep("consume")],
                             exports={"compute": {"symbol": "beta_stage_compute", "decl": decl,
                                                  "decl_sha256": channels.declaration_digest(decl)}})],
            "pipeline": pipeline(["alpha.stage", "beta.stage"], {})}


def topology_base():
    def warp(handle, role, offset):
        return {"domain": "warp", "handle": handle, "extent": {"const": 4, "per": {}}, "align": 1, "offset": offset, "roles": [role]}
    h = lambda owner: {"class": "base", "binding": "bind", "domain": "warp", "owner": owner}
    return {"stages": [stage("alpha.stage", {"load": 4}, claims=[warp("pipelink_warp_load", "load", 0)]),
                       stage("beta.stage", {"mma": 4}, claims=[warp("pipelink_warp_mma", "mma", 4)])],
            "pipeline": pipeline(["alpha.stage", "beta.stage"], {"pipelink_warp_load": h("claim:warp_load"),
                                                                  "pipelink_warp_mma": h("claim:warp_mma")})}


def schema_base():
    variants = [{"key": {"pipelink_depth": 2, "pipelink_variant": 1}, "index": 0},
                {"key": {"pipelink_depth": 4, "pipelink_variant": 1}, "index": 1}]
    return {"stages": [stage("schema.stage", {"load": 4}, variants=variants)]}


def tensor_base():
    """A consumer stage with one tensor import as this linker records it (name, identity, wanted layout, function), the
    site it calls the import from, and three lends of the kinds the reference's corpus uses (test_tensor_contracts.py:68-80:
    relocatable scratch memory, a fixed barrier, fixed registers)."""
    st = stage("tensor.stage", {"epilogue": 4})
    life = {"from": "tile_ready", "to": "import_complete"}
    st["tensor"] = {
        "schema": "tensor-v1", "exports": [],
        "imports": [{"name": "epilogue", "result": "C", "dtype": "fp32", "shape": [128, 32], "layout": "mfma32x32c",
                     "fn": "pipelink_import_accumulator", "sites": ["epilogue_hook"],
                     "lends": [{"name": "scratch", "domain": "smem", "extent": 4096, "align": 128, "scope": "cta", "binding": "relocatable",
                                "location": {"handle": "pipelink_import_scratch", "base": None}, "owner": "epilogue", "lifetime": life},
                               {"name": "rendezvous", "domain": "barrier", "extent": 1, "align": 1, "scope": "cta", "binding": "fixed",
                                "location": {"handle": None, "base": 1}, "owner": "epilogue", "lifetime": life},
                               {"name": "fragment", "domain": "reg", "extent": 32, "align": 1, "scope": "thread", "binding": "fixed",
                                "location": {"handle": "private_fragment", "base": None}, "owner": "epilogue", "lifetime": life}]}],
        "sites": [{"name": "epilogue_hook", "role": "epilogue", "guarantees": ["converged"]}]}
    return {"stages": [st]}


BASES = {"barrier": barrier_base, "double_barrier": double_barrier_base, "call": call_base, "topology": topology_base,
         "schema": schema_base, "tensor": tensor_base, "shared_completion": shared_completion_base, "symbols": symbols_base}


def set_path(root, path, value):
    for p in path[:-1]:
        root = root[p]
    root[path[-1]] = copy.deepcopy(value)


def run_assembly(raw):
    """Load -> validate -> pair -> expand -> solve, as the linker does before code generation."""
    if "tables" in raw:  # the link's symbol check alone, on manifests that carry these tables
        loaded = []
        for stage_id, table in raw["tables"].items():
            m = stage(stage_id, {})
            m["symbols"] = {"defined_strong": list(table["strong"])}
            loaded.append(manifest.load_stage_manifest(m))
        return linker.check_symbols(loaded)
    stages = [manifest.load_stage_manifest(s) for s in raw["stages"]]
    if "pipeline" not in raw:
        return
    pipe = manifest.load_pipeline(raw["pipeline"])
    failures = manifest.validate_assembly(pipe, stages)
    if failures:
        raise LinkError(failures)
    chans = channels.pair_channels(stages)
    exps = channels.expand_all(chans, pipe, stages)
    return pipe, stages, chans, exps, solver.solve(pipe, stages, exps)


@pytest.mark.parametrize("path", sorted(glob.glob(os.path.join(HERE, "golden", "negative", "*.json"))),
                         ids=lambda p: os.path.basename(p)[:-5])
def test_reference_negative_fixture(path):
    case = json.load(open(path))
    raw = BASES[case["base"]]()
    run_assembly(raw)  # the unmutated base is admissible
    mutation = case["mutation"]
    for p in mutation.get("paths", [mutation.get("path")]):
        set_path(raw, p, mutation["value"])
    with pytest.raises(PipeLinkError) as err:
        run_assembly(raw)
    assert err.value.clause_ids == {case["expected_clause"]}
    assert any(case["expected_path"] in f.path for f in err.value.failures), [f.path for f in err.value.failures]
    if case.get("expected_message"):
        assert any(case["expected_message"] in f.message for f in err.value.failures)


def test_shared_completion_expands_to_one_counter_for_three_tiles():
    """The root's completion stands for its own tile and both members'; the members ride the root's slots and arrivals."""
    _, _, _, exps, _ = run_assembly(shared_completion_base())
    by = {e.channel: e for e in exps}
    assert by["root"].tx_full == 4 * 4 * 2 + 2 * (2 * 2 * 2) and by["root"].detail == {}
    for m in ("member", "leaf"):
        assert by[m].tx_full == 2 * 2 * 2 and by[m].detail == {"member_of": {"full": "root"}}
        assert by[m].slots == by["root"].slots and by[m].arrive_full == by["root"].arrive_full


def gallery():
    """A producer/consumer ring like the reference's contract gallery (T3): stage ids and channel
    names chosen so that the diagnostics read exactly as its tutorial prints them."""
    full = {"slots": "pipelink_ring_full", "arrive": {"count": 1, "by": "producer"}, "tx_bytes": "tile"}

    def ep(direction, role):
        e = ring_endpoint("tile_ring", direction, role, full, shape=(64, 128), stride=16384)
        e["ring"]["depth"]["handle"] = "pipelink_ring_depth"
        e["protocol"]["empty"] = {"slots": "pipelink_ring_empty", "arrive": {"count": "threads(consumer)", "by": "consumer"}, "tx_bytes": 0}
        e["protocol"]["init"] = {"owner": "producer", "materializer": "dispatch", "phase": 0}
        e["binds"] = {"full": "pipelink_ring_full", "empty": "pipelink_ring_empty"}
        return e
    slot = lambda h: {"domain": "mbarrier", "handle": h, "extent": {"const": 0, "per": {"pipelink_ring_depth": 1}}, "align": 1}
    tiles = {"domain": "smem", "handle": "pipelink_ring_tiles", "extent": {"const": 0, "per": {"pipelink_ring_depth": 16384}}, "align": 128}
    wclaim = lambda h, role, off, n: {"domain": "warp", "handle": h, "extent": {"const": n, "per": {}}, "align": 1, "offset": off, "roles": [role]}
    handles = {"pipelink_ring_depth": {"class": "depth", "binding": "bind", "values": [2, 4], "owner": "channel:tile_ring"},
               "pipelink_ring_full": {"class": "base", "binding": "bind", "domain": "mbarrier", "owner": "claim:full"},
               "pipelink_ring_empty": {"class": "base", "binding": "bind", "domain": "mbarrier", "owner": "claim:empty"},
               "pipelink_ring_tiles": {"class": "base", "binding": "bind", "domain": "smem", "owner": "claim:tiles"},
               "pipelink_ring_warp_producer": {"class": "base", "binding": "bind", "domain": "warp", "owner": "claim:wp"},
               "pipelink_ring_warp_consumer": {"class": "base", "binding": "bind", "domain": "warp", "owner": "claim:wc"}}
    return {"stages": [stage("org.ring.producer", {"producer": 1}, endpoints=[ep("produce", "producer")],
                             claims=[slot("pipelink_ring_full"), slot("pipelink_ring_empty"), tiles,
                                     wclaim("pipelink_ring_warp_producer", "producer", 0, 1)], params=(256, 128)),
                       stage("org.ring.consumer", {"consumer": 4}, endpoints=[ep("consume", "consumer")],
                             claims=[wclaim("pipelink_ring_warp_consumer", "consumer", 1, 4)], params=(24, 8))],
            "pipeline": pipeline(["org.ring.consumer", "org.ring.producer"], handles)}


def test_gallery_known_answers_ring_depth_threads_params():
    # examples/ring-pipeline/README.md:31 -- threads 160; dyn smem 32832 (depth 2) / 65664 (depth 4); params 384
    raw = gallery()
    pipe, stages, chans, exps, sol = run_assembly(raw)
    assert sol.value("pipelink_ring_depth") == 4 and sol.dyn_smem_bytes == 4 * 16384 + 8 * 16 == 65664
    assert sol.threads == (1 + 4) * 32 == 160
    layout = glue.params_layout(pipe, stages)
    assert layout["total_bytes"] == 384
    assert [(e["stage_id"], e["offset"]) for e in layout["entries"]] == [("org.ring.consumer", 0), ("org.ring.producer", 128)]
    raw["pipeline"]["pipeline"]["forced_bindings"] = {"pipelink_ring_depth": 2}
    sol2 = run_assembly(raw)[4]
    assert sol2.value("pipelink_ring_depth") == 2 and sol2.dyn_smem_bytes == 2 * 16384 + 4 * 16 == 32832
    exp = exps[0]
    assert (exp.tx_full, exp.arrive_full, exp.arrive_empty) == (64 * 128 * 2, 1, 128)
    # the same assembly retargeted to gfx950: a warp is a 64-lane wave
    for s in raw["stages"]:
        s["pipelink_abi"] = abi("gfx950")
    raw["pipeline"]["pipelink_abi"] = abi("gfx950")
    sol3 = run_assembly(raw)[4]
    assert sol3.threads == 5 * 64 and sol3.dyn_smem_bytes == 32832


GALLERY_CASES = [
    ("L-PROTO", lambda r: set_path(r, ["stages", 1, "endpoints", 0, "protocol", "full", "arrive", "count"], 2),
     "[L-PROTO] channels.tile_ring.protocol.full.arrive: producer and consumer arrival declarations disagree"),
    ("L-TOPO", lambda r: set_path(r, ["stages", 1, "topology", "persistent"], True),
     "[L-TOPO] stages.org.ring.consumer.topology.persistent: stage and pipeline persistence disagree"),
    ("L-HANDLE", lambda r: set_path(r, ["stages", 1, "endpoints", 0, "ring", "depth", "handle"], "pipelink_ring_deph"),
     "[L-HANDLE] stages.org.ring.consumer.endpoints.tile_ring.ring.depth.handle: referenced pipelink_* handle is not declared in pipeline scope"),
    ("L-PHASE", lambda r: set_path(r, ["stages", 1, "claims", 0, "lifetime"], "phase:stedy"),
     "[L-PHASE] stages.org.ring.consumer.claims.warp.pipelink_ring_warp_consumer.lifetime: claim lifetime names an undeclared phase"),
]


@pytest.mark.parametrize("clause,mutate,line", GALLERY_CASES, ids=[c[0] for c in GALLERY_CASES])
def test_contract_gallery_diagnostics_verbatim(clause, mutate, line):
    # docs/tutorials/T3-contract-gallery.md:92-94,105-107,118-120,164-166
    raw = gallery()
    mutate(raw)
    with pytest.raises(PipeLinkError) as err:
        run_assembly(raw)
    assert clause in err.value.clause_ids
    assert line in str(err.value)


def test_aggregate_params_overflow_is_l_params():
    # docs/tutorials/T3-contract-gallery.md:150-152: each blob under the limit, the sum above it
    raw = gallery()
    raw["stages"][1]["params"]["bytes"] = 32640 + 24
    pipe, stages = run_assembly(raw)[:2]
    with pytest.raises(LinkError) as err:
        glue.params_layout(pipe, stages)
    assert "[L-PARAMS] params.total_bytes: aggregate parameter layout exceeds the target parameter limit" in str(err.value)


def test_depth_that_does_not_fit_falls_back_and_forced_overflow_is_l_overlap():
    raw = gallery()
    raw["stages"][0]["claims"][2]["extent"]["per"]["pipelink_ring_depth"] = 100000   # 4 stages > LDS, 2 fit
    sol = run_assembly(raw)[4]
    assert sol.value("pipelink_ring_depth") == 2
    raw["pipeline"]["pipeline"]["forced_bindings"] = {"pipelink_ring_depth": 4}
    with pytest.raises(SolveError) as err:
        run_assembly(raw)
    assert err.value.clause_ids == {"L-OVERLAP"} and "no feasible joint binding and placement exists" in str(err.value)


def test_protocol_mismatch_classes_all_raise_l_proto():
    # the classes enumerated in pipec/tests/pipec2/test_protocol.py:439-478
    muts = {
        "kind": (["stages", 1, "endpoints", 0, "protocol", "kind"], "call", "protocol.kind"),
        "ring": (["stages", 1, "endpoints", 0, "ring", "stage_stride_bytes"], 64, ".ring"),
        "release": (["stages", 1, "endpoints", 0, "protocol", "release"], "never", "protocol.release"),
        "slots": (["stages", 1, "endpoints", 0, "protocol", "empty", "slots"], "pipelink_full", "protocol.empty.slots"),
        "by": (["stages", 1, "endpoints", 0, "protocol", "full", "arrive", "by"], "mma", "protocol.full.arrive"),
        "tx": (["stages", 1, "endpoints", 0, "protocol", "full", "tx_bytes"], 16, "protocol.full.tx_bytes"),
        "init": (["stages", 1, "endpoints", 0, "protocol", "init", "owner"], "mma", "protocol.init"),
        "count0": (["stages", 0, "endpoints", 0, "protocol", "empty", "arrive", "count"], "threads(ghost)", "arrive"),
    }
    for name, (path, value, where) in muts.items():
        raw = barrier_base()
        set_path(raw, path, value)
        with pytest.raises(PipeLinkError) as err:
            run_assembly(raw)
        assert "L-PROTO" in err.value.clause_ids, name
        assert any(where in f.path for f in err.value.failures), (name, [f.path for f in err.value.failures])


def test_pairing_failures_are_l_pair_and_l8():
    raw = barrier_base()
    raw["stages"][1]["endpoints"] = []
    with pytest.raises(LinkError) as err:
        run_assembly(raw)
    assert err.value.clause_ids == {"L-PAIR"}
    raw = barrier_base()
    raw["stages"][1]["endpoints"][0]["layout"]["stride"] = [[8], [1]]
    with pytest.raises(LinkError) as err:
        run_assembly(raw)
    assert err.value.clause_ids == {"L8"}


def test_solver_is_deterministic_under_input_permutation():
    base = run_assembly(gallery())[4].to_json_obj()
    for perm in itertools.permutations(range(4)):
        raw = gallery()
        raw["stages"][0]["claims"] = [raw["stages"][0]["claims"][i] for i in perm]
        raw["pipeline"]["pipeline"]["handles"] = dict(reversed(list(raw["pipeline"]["pipeline"]["handles"].items())))
        assert run_assembly(raw)[4].to_json_obj() == base


def test_phase_exclusive_claims_share_lds():
    raw = gallery()
    raw["pipeline"]["pipeline"]["phases"] = ["steady", "drain"]
    raw["pipeline"]["pipeline"]["exclusive"] = [["steady", "drain"]]
    raw["pipeline"]["pipeline"]["handles"]["pipelink_ring_scratch"] = {"class": "base", "binding": "bind", "domain": "smem", "owner": "claim:s"}
    raw["stages"][0]["claims"][2]["lifetime"] = "phase:steady"
    raw["stages"][0]["claims"].append({"domain": "smem", "handle": "pipelink_ring_scratch", "extent": {"const": 60000, "per": {}},
                                       "align": 16, "lifetime": "phase:drain"})
    sol = run_assembly(raw)[4]
    assert sol.dyn_smem_bytes == 65664   # the drain-phase scratch overlays the steady-phase ring
    raw["pipeline"]["pipeline"]["exclusive"] = []
    assert run_assembly(raw)[4].dyn_smem_bytes > 65664 + 59000


def test_clause_registry_and_error_format():
    for cid in ("L-PROTO", "L-HANDLE", "L-PHASE", "L-TOPO", "L-PARAMS", "L-OVERLAP", "L-PAIR", "L8", "P-CONTAINER"):
        assert cid in CLAUSES
    with pytest.raises(ValueError):
        ClauseFailure("L-NOPE", "x", "y")
    with pytest.raises(ValueError):
        register_clause("L-PROTO", phase="protocol")
    err = SchemaError([ClauseFailure("L-PROTO", "b", "two"), ClauseFailure("L-HANDLE", "a", "one")])
    assert str(err) == "[L-HANDLE] a: one; [L-PROTO] b: two"


def test_declaration_digest_ignores_comments_and_whitespace_only():
    a = 'extern "C" int f(int value);'
    assert channels.declaration_digest(a) == channels.declaration_digest('extern "C"   int f(int /*x*/ value); // trailing')
    assert channels.declaration_digest(a) != channels.declaration_digest('extern "C" int f(long value);')
    # the digest the reference's fixture 06 records for its mutated declaration
    assert channels.declaration_digest('extern "C" int beta_stage_compute(long value);') == \
        "61728d8dafdbfbfc7641e14117420c9e1b930904f889859b9dcb6b20807d1fdb"
