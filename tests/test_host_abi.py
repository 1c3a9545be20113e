"""Host ABI v2: the providers' abi / query / build / release against the broker's mirrors, without a GPU.

Pins (reference: pipec/src/pipec2/host/include/pipelink_host_abi_v2.h:21-28,43-47,293-300 and
campaigns/mok/port/gemm/provider.cu:217-303): version and struct_bytes checks, status codes,
capacity rules, caller-owned residue bytes, null-session release, and that the params image the
broker assembles through the providers is byte-identical to the one the forward entry builds."""
import ctypes
import json
import os
from ctypes import byref, sizeof

import pytest

from pipelink_amd.host import broker
from pipelink_amd.host.backend import PlkError, load_library

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

SCALARS = {"mok.num_local_tokens": 512, "mok.hidden": 320, "mok.intermediate": 192, "mok.num_local_experts": 4,
           "mok.swiglu_limit": 7.0, "mok.pass": 1, "mok.precision": 1, "mok.routed_rows": 1024, "mok.ld_q_h": 384,
           "mok.ld_q_i": 256, "mok.ld_sc_h": 16, "mok.ld_sc_i": 16,
           "mok.workspace_words": 32 + 1024 // 256 + 4}   # status and counter words + one counter per possible row tile
# the owner inventory is what the built pipeline's link recorded from the stages' PL_HOST_* declarations
_LINK_JSON = os.path.join(ROOT, "pipelink_amd", "stages", "mok", "build", "link", "link.json")
if not os.path.exists(_LINK_JSON):
    pytest.skip("the routed-expert FFN cell is not built (run __graft_entry__.build()): " + _LINK_JSON, allow_module_level=True)
_BUILT = json.loads(open(_LINK_JSON).read())
HOST = _BUILT["host"]
LINK = {"threads": 256, "dyn_smem_bytes": _BUILT["dyn_smem_bytes"], "kernel_symbol": "pipelink_kernel", "workgroups_per_cu": 1,
        "host": HOST, "params": _BUILT["params"]}
_AT = {e["stage_id"]: (e["offset"], e["offset"] + e["bytes"]) for e in LINK["params"]["entries"]}
FW, GEMM, ACT = _AT["mok.framework"], _AT["mok.gemm"], _AT["mok.act"]
GROUPS = {g["owner"]: g for g in HOST["groups"]}


def _resources(scalars=SCALARS, row_token=True):
    """Fake device addresses (nothing is dereferenced on the host): 1 MiB apart, 256-byte aligned."""
    out, addr = {}, 0x7F0000000000
    for stage, chans in broker.channel_shapes(LINK, scalars).items():
        out[stage] = {}
        for name, (bits, _, extents) in chans.items():
            if name == "row_token" and not row_token:
                continue
            size = bits // 8
            for e in extents:
                size *= e
            out[stage][name] = broker.Resource(addr, size)
            addr += 1 << 24
    return out


def test_abi_report_matches_the_ctypes_mirrors():
    lib = load_library()
    assert set(GROUPS) == {"mok.framework", "mok.gemm", "mok.act"}
    for stage, group in GROUPS.items():
        rep = broker.Owner(lib, group).report()          # raises on any size / alignment / digest mismatch
        assert rep.entry_count == 20 + len(group["provider"]["abi_types"])
    assert sizeof(broker.MokGemmResidue) == 264 and sizeof(broker.MokActResidue) == 40 and sizeof(broker.MokFrameworkParams) == 32
    assert (FW, GEMM, ACT) == ((0, 32), (32, 296), (296, 336))


def test_abi_report_rejects_wrong_version_capacity_and_ids():
    lib = load_library()
    owner = broker.Owner(lib, GROUPS["mok.gemm"])
    rep = broker.AbiReport()
    rep.header = broker.Header(3, sizeof(rep))
    assert owner.abi(byref(rep)) == 1                     # PLK_E_VERSION
    rep.header = broker.Header(2, sizeof(rep) - 8)
    assert owner.abi(byref(rep)) == 1
    rep.header = broker.Header(2, sizeof(rep))
    entries = (broker.LayoutEntry * 22)()
    rep.entries, rep.entry_capacity = entries, 21
    assert owner.abi(byref(rep)) == 2                     # PLK_E_CAPACITY
    rep.entry_capacity = 22
    assert owner.abi(byref(rep)) == 4                     # PLK_E_CONTRACT: ids not pre-filled


def test_plan_builds_the_same_image_as_the_structs_say():
    res = _resources()
    image, geometry, owners = broker.plan(LINK, res, SCALARS, compute_units=256)
    assert len(image) == 336 and geometry["block"] == (256, 1, 1) and geometry["dyn_lds"] == LINK["dyn_smem_bytes"]
    assert geometry["grid"][0] % 8 == 0 and 0 < geometry["grid"][0] <= 256
    fw = broker.MokFrameworkParams.from_buffer_copy(image[FW[0]:FW[1]])
    g = broker.MokGemmResidue.from_buffer_copy(image[GEMM[0]:GEMM[1]])
    a = broker.MokActResidue.from_buffer_copy(image[ACT[0]:ACT[1]])
    assert fw.tokens_per_expert == res["mok.framework"]["tokens_per_expert"].address
    assert fw.workspace == res["mok.framework"]["workspace"].address
    # gate/up: ceil(192 / 128) column tiles, down: ceil(320 / 256)
    assert (fw.num_experts, fw.op, fw.num_col_tiles_gate_up, fw.num_col_tiles_down) == (4, 3, 2, 2)
    assert (g.x.q, g.x.rows, g.x.k, g.x.ld_q, g.x.ld_sc) == (res["mok.gemm"]["x_q"].address, 512, 320, 384, 16)
    assert (g.w_gate.rows, g.w_gate.k, g.w_gate.ld_q, g.w_gate.expert_pitch_q, g.w_gate.expert_pitch_sc) == \
        (192, 320, 64, 192 * 320, 3 * 192 * 4)
    assert (g.w_down.rows, g.w_down.k, g.w_down.expert_pitch_q) == (320, 192, 320 * 192)
    assert (g.hidden.rows, g.hidden.ld_q, g.y, g.ld_y) == (1024, 256, res["mok.gemm"]["y"].address, 320)
    assert g.row_token == res["mok.gemm"]["row_token"].address
    assert (a.rows, a.cols, a.ld_q, a.ld_sc, a.swiglu_limit) == (1024, 192, 256, 16, 7.0)
    for o in reversed(owners):
        assert o.release(o.session) == 0                  # null sessions release fine
    down = dict(SCALARS, **{"mok.pass": 2})
    image2, _, _ = broker.plan(LINK, res, down, compute_units=256)
    fw2 = broker.MokFrameworkParams.from_buffer_copy(image2[FW[0]:FW[1]])
    assert fw2.op == 5 and image2[FW[1]:] == image[FW[1]:]
    # both GEMMs in one launch: op 0, and only with rows of `hidden` that are whole cache lines
    both, _, _ = broker.plan(LINK, res, dict(SCALARS, **{"mok.pass": 0}), compute_units=256)
    assert broker.MokFrameworkParams.from_buffer_copy(both[FW[0]:FW[1]]).op == 0 and both[FW[1]:] == image[FW[1]:]
    with pytest.raises(PlkError) as err:
        odd = dict(SCALARS, **{"mok.pass": 0, "mok.ld_q_i": 192})
        broker.plan(LINK, _resources(odd), odd, compute_units=256)
    assert err.value.status == 3


def test_optional_row_token_channel_may_be_absent():
    res = _resources(row_token=False)
    image, _, _ = broker.plan(LINK, res, SCALARS, compute_units=256)
    assert broker.MokGemmResidue.from_buffer_copy(image[GEMM[0]:GEMM[1]]).row_token is None


@pytest.mark.parametrize("mutate,status", [
    (lambda s, r, l: s.update({"mok.hidden": 96}), 3),                     # not a multiple of 64: PLK_E_ARGUMENT
    (lambda s, r, l: s.pop("mok.routed_rows"), 3),                         # a scalar is missing
    (lambda s, r, l: s.update({"mok.precision": 2}), 3),                   # only MXFP8 is built
    (lambda s, r, l: l.update(threads=512), 4),                            # block shape: PLK_E_CONTRACT
    (lambda s, r, l: r["mok.gemm"].update(y=broker.Resource(r["mok.gemm"]["y"].address, 16)), 5),   # too small
    (lambda s, r, l: r["mok.gemm"].update(x_q=broker.Resource(r["mok.gemm"]["x_q"].address + 4,
                                                              r["mok.gemm"]["x_q"].allocation_bytes)), 5),  # misaligned
    (lambda s, r, l: l["params"]["entries"][1].update(bytes=128), 2),      # residue capacity: PLK_E_CAPACITY
])
def test_provider_and_broker_reject_bad_inputs(mutate, status):
    scalars, res, link = dict(SCALARS), _resources(), json.loads(json.dumps(LINK))
    mutate(scalars, res, link)
    with pytest.raises(PlkError) as err:
        broker.plan(link, res, scalars, compute_units=256)
    assert err.value.status == status


def test_build_checks_the_resource_records_itself():
    """Call build directly with a resource smaller than the demand: PLK_E_RESOURCE, and no session."""
    lib = load_library()
    owner = broker.Owner(lib, GROUPS["mok.act"])
    shared = broker._Scalars(SCALARS, HOST["scalars"])
    common = broker.Common()
    common.header = broker.Header(2, sizeof(common))
    common.channel_count, common.shared = 2, shared.pointer
    common.block, common.cluster = broker.Dim3(256, 1, 1), broker.Dim3(1, 1, 1)
    devres = (broker.DeviceResource * 2)(broker.DeviceResource(1, 2, 0x1000, 64, 0, 0, 0, None, 0),
                                         broker.DeviceResource(2, 2, 0x2000, 1 << 20, 0, 0, 0, None, 0))
    r = broker.Resources()
    r.header = broker.Header(2, sizeof(r))
    r.channel_count, r.channels, r.shared = 2, devres, shared.pointer
    out = ctypes.create_string_buffer(40)
    session = ctypes.c_void_p(123)
    assert owner.build(byref(common), None, byref(r), out, 40, None, 0, byref(session)) == 5
    assert session.value is None
    assert owner.build(byref(common), None, byref(r), out, 40, None, 1, byref(session)) == 2      # transfers are not reported
    assert owner.build(byref(common), ctypes.c_void_p(1), byref(r), out, 40, None, 0, byref(session)) == 3   # args must be null
    assert owner.release(ctypes.c_void_p(1)) == 7 and owner.release(None) == 0


def test_owner_inventory_comes_from_the_link():
    """What the stages declared with PL_HOST_* is what the link recorded and the broker works from."""
    assert HOST["protocol"] == 2 and HOST["params"]["blobs"] == []
    gemm = GROUPS["mok.gemm"]
    assert gemm["params_group"] == "mok.gemm.params" and gemm["provider"]["symbols"]["build"] == "pipelink_params_build_mok_gemm"
    assert [c["name"] for c in gemm["channels"]] == ["x_q", "x_sc", "w_gate_q", "w_gate_sc", "w_up_q", "w_up_sc", "w_down_q",
                                                     "w_down_sc", "hidden_q", "hidden_sc", "y", "row_token"]
    assert [c["name"] for c in gemm["channels"] if c["optional"]] == ["row_token"]
    assert {t["name"]: t["bytes"] for t in gemm["provider"]["abi_types"]} == {"MokGemmResidue": 264, "MokMxView": 48}
    assert [s["id"] for s in HOST["scalars"]] == [1, 2, 3, 4, 10, 11, 12, 60, 61, 62, 63, 64, 65]
    assert [c["name"] for c in GROUPS["mok.framework"]["channels"]] == ["tokens_per_expert", "workspace"]
    assert broker.evaluate_extents("mok.num_local_experts, floor(mok.hidden,64), ceil(mok.intermediate, 128), 4", SCALARS) == (4, 5, 2, 4)
    with pytest.raises(PlkError):
        broker.evaluate_extents("mok.hidden * 2", SCALARS)


def test_broker_refuses_a_link_without_inventory_or_with_foreign_records():
    res = _resources()
    bare = {k: v for k, v in LINK.items() if k != "host"}
    with pytest.raises(PlkError) as err:
        broker.plan(bare, res, SCALARS, compute_units=256)
    assert err.value.status == 4 and "host section" in str(err.value)
    other = json.loads(json.dumps(LINK))
    other["host"]["groups"][0]["provider"]["abi_types"][0]["bytes"] += 8       # a record this broker mirrors differently
    with pytest.raises(PlkError) as err:
        broker.plan(other, res, SCALARS, compute_units=256)
    assert err.value.status == 1
    gone = json.loads(json.dumps(LINK))
    gone["host"]["groups"][1]["provider"]["symbols"]["query"] = "pipelink_params_query_nobody"
    with pytest.raises(PlkError) as err:
        broker.plan(gone, res, SCALARS, compute_units=256)
    assert err.value.status == 4 and "missing provider export" in str(err.value)


def test_fixture_owns_buffers_until_it_closes():
    """pipec2.host.fixture.Fixture's contract (fixture.py:44-96 in the reference) on a host-memory backend."""
    from pipelink_amd.host.fixture import Domain, Fixture

    class Memory:
        lost = False

        def __init__(self):
            self.mem, self.next, self.freed, self.synced = {}, 0x1000, [], 0

        def allocate(self, size, align=256):
            addr, self.next = self.next, self.next + (size + 255) // 256 * 256
            self.mem[addr] = bytearray(size)
            return addr

        def free(self, addr): self.freed.append(addr)
        def upload(self, addr, data, stream=None): self.mem[addr][:len(data)] = data
        def zero(self, addr, size, stream=None): self.mem[addr][:size] = bytes(size)
        def readback(self, addr, size, stream=None): return bytes(self.mem[addr][:size])
        def synchronize(self, stream=None): self.synced += 1

    be = Memory()
    with Fixture(be) as fx:
        a = fx.tensor("a", data=b"\x01\x02\x03\x04", allocation_bytes=4)
        out = fx.tensor("out", data=None, allocation_bytes=8, output=True)
        assert (a.address, a.allocation_bytes) == (0x1000, 4) and out.address == 0x1100
        with pytest.raises(ValueError):
            fx.tensor("a", data=None, allocation_bytes=4)              # a name is lent once
        with pytest.raises(ValueError):
            fx.tensor("b", data=b"\x00", allocation_bytes=4)           # data must cover the allocation
        be.mem[out.address][:] = b"ABCDEFGH"
        assert fx.readback() == {"out": b"ABCDEFGH"}
    assert be.freed == [0x1100, 0x1000] and be.synced == 1            # reverse order, after a drain
    lost = Memory()
    lost.lost = True
    with Fixture(lost) as fx:
        fx.tensor("a", data=None, allocation_bytes=4)
    assert lost.freed == []                                           # an abandoned backend's memory is not reused
    assert Domain(0, 1).world == 1


def test_launch_verb_takes_a_host_link_through_its_providers(tmp_path):
    """`pipec launch` on a link with a host section (cli.py:226-258, launcher.py:284-333 in the reference): the
    argument checks that need no GPU."""
    from pipelink_amd.pipec import cli, launcher
    from pipelink_amd.pipec.clauses import LaunchError
    from pipelink_amd.host.fixture import Fixture, load_inputs

    link_path = _LINK_JSON
    with pytest.raises(LaunchError) as err:
        launcher.launch(link_path, grid=(8,))
    assert err.value.failures[0].path == "launch.host"                        # host-less arguments on a host link
    with pytest.raises(LaunchError) as err:
        launcher.launch(link_path, grid=None, providers={"mok.gemm.params": "x.so"})
    assert err.value.failures[0].path == "launch.host_inputs"
    inputs = tmp_path / "inputs.json"
    inputs.write_text(json.dumps({"scalars": {}, "resources": {}}))
    with pytest.raises(LaunchError) as err:
        launcher.launch(link_path, grid=None, providers={"mok.gemm.params": "x.so"}, host_inputs=inputs)
    assert err.value.clause_ids == {"L-HOSTABI"} and err.value.failures[0].detail["expected"] == [
        "mok.act.params", "mok.framework.params", "mok.gemm.params"]
    assert cli.main(["launch", link_path, "--provider", "mok.gemm.params=x.so", "--host-inputs", str(inputs)]) == 1

    class Memory:
        lost = False
        def __init__(self): self.mem, self.next = {}, 0x1000
        def allocate(self, size, align=256):
            addr, self.next = self.next, self.next + (size + 255) // 256 * 256
            self.mem[addr] = bytearray(size)
            return addr
        def free(self, addr): pass
        def upload(self, addr, data, stream=None): self.mem[addr][:len(data)] = data
        def zero(self, addr, size, stream=None): pass
        def readback(self, addr, size, stream=None): return bytes(self.mem[addr][:size])
        def synchronize(self, stream=None): pass

    (tmp_path / "x.bin").write_bytes(b"\x05" * 16)
    inputs.write_text(json.dumps({"scalars": {"mok.hidden": 64}, "resources": {
        "x_q": {"data": "x.bin", "allocation_bytes": 16, "extents": [1, 16], "bit_strides": [128, 8], "dtype_id": 1, "alignment": 16,
                "origin_byte_offset": 0, "origin_bit_offset": 0},
        "y": {"data": None, "allocation_bytes": 32, "output": "y.bin"}}}))
    with Fixture(Memory()) as fx:
        scalars, outputs = load_inputs(inputs, fx)
        assert scalars == {"mok.hidden": 64} and outputs == {"y": tmp_path / "y.bin"}
        assert fx.resources["x_q"].allocation_bytes == 16 and fx.backend.mem[fx.resources["x_q"].address] == b"\x05" * 16
        assert set(fx.readback()) == {"y"}
    inputs.write_text(json.dumps({"scalars": {}, "resources": {"x_q": {"data": None}}}))
    with pytest.raises(ValueError), Fixture(Memory()) as fx:
        load_inputs(inputs, fx)
