"""Broker side of the PipeLink host ABI v2: report / query / build each owner once, assemble the
params image at the linked offsets, launch.

Plays the part of ``pipec2.host.broker.open_host`` (pipec/src/pipec2/host/broker.py:804-949) for
the routed-expert FFN pipeline: the owners' providers (``pipelink_params_{abi,query,build,
release}_<suffix>``, include/plk_host_abi_v2.h) live in the C-ABI library; the broker owns every
record, array and the residue bytes, checks each provider's answers against what the caller
holds, and releases sessions in reverse build order (broker.py:768-801).  The owner inventory
comes from the ``host`` section of link.json (broker.py:818-830): per params group the provider's
entry points, the record types it must report, its scalars and its caller-owned channels with
their extents as expressions over the scalars -- the stages declared them (``PL_HOST_*``), the
link gathered them.  This side only keeps the ctypes mirrors of the record types, by C name.

Pure ctypes; nothing here needs a GPU until ``HostSession.launch``."""
from __future__ import annotations

import ctypes
import hashlib
import re
import struct
from ctypes import (POINTER, Structure, byref, c_int64, c_size_t, c_uint8, c_uint32, c_uint64, c_void_p, cast, pointer,
                    sizeof)
from dataclasses import dataclass
from typing import Any, Mapping

from .fixture import Domain, Fixture, Resource  # noqa: F401  (the reference exposes them beside open_host)
from .backend import PlkError, load_library

ABI_V2 = 2
SCALAR_I64, SCALAR_F64 = 2, 3
ACCESS_READ, ACCESS_WRITE = 1, 2


# ---- record mirrors (member order = include/plk_host_abi_v2.h) -----------------------------------
class Header(Structure):
    _fields_ = [("abi_version", c_uint32), ("struct_bytes", c_uint32)]


class Digest(Structure):
    _fields_ = [("sha256", c_uint8 * 32)]


class ProfileDigest(Structure):
    _fields_ = [("dtypes", Digest)]


class Dim3(Structure):
    _fields_ = [("x", c_uint32), ("y", c_uint32), ("z", c_uint32)]


class Scalar(Structure):
    _fields_ = [("scalar_id", c_uint32), ("scalar_type", c_uint32), ("value_bits", c_uint64)]


class SharedScalars(Structure):
    _fields_ = [("header", Header), ("image_bytes", c_uint64), ("record_count", c_uint32), ("record_offset", c_uint32)]


class TensorMeta(Structure):
    _fields_ = [("channel_id", c_uint32), ("dtype_id", c_uint32), ("rank", c_uint32), ("access", c_uint32),
                ("allocation_bytes", c_uint64), ("alignment_bytes", c_uint64), ("origin_byte_offset", c_uint64),
                ("origin_bit_offset", c_uint32), ("reserved", c_uint32), ("extents", POINTER(c_uint64)),
                ("bit_strides", POINTER(c_int64))]


class Geometry(Structure):
    _fields_ = [("geometry_present", c_uint32), ("launch_required", c_uint32), ("grid", Dim3), ("block", Dim3),
                ("cluster", Dim3), ("reserved", c_uint32), ("dynamic_smem_bytes", c_uint64)]


class DomainRecord(Structure):  # plk_domain_v2 (the caller-facing Domain tuple is the fixture module's)
    _fields_ = [("domain_id", c_uint32), ("rank", c_uint32), ("world", c_uint32), ("reserved", c_uint32)]


class Common(Structure):
    _fields_ = [("header", Header), ("owner_id", c_uint32), ("channel_count", c_uint32), ("domain_count", c_uint32),
                ("reserved", c_uint32), ("shared", POINTER(SharedScalars)), ("channels", POINTER(TensorMeta)),
                ("domains", POINTER(DomainRecord)), ("block", Dim3), ("cluster", Dim3), ("dynamic_smem_bytes", c_uint64),
                ("profile", ProfileDigest), ("owner_contract", Digest)]


class ChannelDemand(Structure):
    _fields_ = [("channel_id", c_uint32), ("dtype_id", c_uint32), ("rank", c_uint32), ("access", c_uint32),
                ("minimum_allocation_bytes", c_uint64), ("alignment_bytes", c_uint64), ("extents", POINTER(c_uint64)),
                ("bit_strides", POINTER(c_int64))]


class WorkspaceDemand(Structure):
    _fields_ = [("workspace_id", c_uint32), ("reserved", c_uint32), ("bytes", c_uint64), ("alignment_bytes", c_uint64)]


class Demands(Structure):
    _fields_ = [("header", Header), ("channel_count", c_uint32), ("channel_capacity", c_uint32),
                ("channels", POINTER(ChannelDemand)), ("workspace_count", c_uint32), ("workspace_capacity", c_uint32),
                ("workspaces", POINTER(WorkspaceDemand)), ("geometry", Geometry)]


class DeviceResource(Structure):
    _fields_ = [("channel_id", c_uint32), ("access", c_uint32), ("allocation_address", c_uint64),
                ("allocation_bytes", c_uint64), ("origin_byte_offset", c_uint64), ("origin_bit_offset", c_uint32),
                ("domain_id", c_uint32), ("peer_addresses", POINTER(c_uint64)), ("multicast_address", c_uint64)]


class WorkspaceResource(Structure):
    _fields_ = [("workspace_id", c_uint32), ("reserved", c_uint32), ("device_address", c_uint64), ("bytes", c_uint64),
                ("alignment_bytes", c_uint64)]


class Resources(Structure):
    _fields_ = [("header", Header), ("channel_count", c_uint32), ("workspace_count", c_uint32),
                ("channels", POINTER(DeviceResource)), ("workspaces", POINTER(WorkspaceResource)),
                ("shared", POINTER(SharedScalars)), ("cuda_stream_token", c_uint64), ("geometry", Geometry)]


class TmaTiledDetail(Structure):
    _fields_ = [("swizzle", c_uint32), ("rank", c_uint32), ("box_elements", c_uint64 * 5),
                ("element_strides", c_uint32 * 5), ("reserved", c_uint32)]


class TransferReport(Structure):
    _fields_ = [("transfer_id", c_uint32), ("access", c_uint32), ("residue_offset", c_uint64),
                ("representation_bytes", c_uint64), ("representation_align", c_uint64), ("storage_dtype_id", c_uint32),
                ("ring_depth", c_uint32), ("ring_stage_stride_bytes", c_uint64), ("footprint_bytes_per_stage", c_uint64),
                ("credit_bytes_per_stage", c_uint64), ("source_origin_bits", c_uint64), ("source_span_bits", c_uint64),
                ("vendor_kind", c_uint32), ("reserved", c_uint32), ("vendor_detail", c_void_p)]


class LayoutEntry(Structure):
    _fields_ = [("abi_type_id", c_uint32), ("reserved", c_uint32), ("bytes", c_uint64), ("alignment_bytes", c_uint64),
                ("compiler_layout", Digest)]


class AbiReport(Structure):
    _fields_ = [("header", Header), ("entry_count", c_uint32), ("entry_capacity", c_uint32),
                ("entries", POINTER(LayoutEntry)), ("profile", ProfileDigest), ("owner_contract", Digest)]


# owner records (pipelink_amd/stages/mok/include/mok_abi.h)
class MokMxView(Structure):
    _fields_ = [("q", c_void_p), ("sc", c_void_p), ("expert_pitch_q", c_int64), ("expert_pitch_sc", c_int64),
                ("rows", ctypes.c_int32), ("k", ctypes.c_int32), ("ld_q", ctypes.c_int32), ("ld_sc", ctypes.c_int32)]


class MokGemmResidue(Structure):
    _fields_ = [("x", MokMxView), ("hidden", MokMxView), ("w_gate", MokMxView), ("w_up", MokMxView),
                ("w_down", MokMxView), ("row_token", c_void_p), ("y", c_void_p), ("ld_y", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


class MokActResidue(Structure):
    _fields_ = [("hidden_q", c_void_p), ("hidden_sc", c_void_p), ("rows", ctypes.c_int32), ("cols", ctypes.c_int32),
                ("ld_q", ctypes.c_int32), ("ld_sc", ctypes.c_int32), ("swiglu_limit", ctypes.c_float),
                ("reserved", ctypes.c_int32)]


class MokFrameworkParams(Structure):
    _fields_ = [("tokens_per_expert", c_void_p), ("workspace", c_void_p),
                ("num_experts", ctypes.c_int32), ("op", ctypes.c_int32), ("num_col_tiles_gate_up", ctypes.c_int32),
                ("num_col_tiles_down", ctypes.c_int32)]


# neutral inventory, in the order the providers report it (type id, C name, mirror)
NEUTRAL_TYPES = [
    (0x70000001, "plk_abi_report_v2", AbiReport), (0x70000002, "plk_channel_demand_v2", ChannelDemand),
    (0x70000003, "plk_common_v2", Common), (0x70000004, "plk_demands_v2", Demands),
    (0x70000005, "plk_tma_tiled_detail_v2", TmaTiledDetail), (0x70000006, "plk_device_resource_v2", DeviceResource),
    (0x70000007, "plk_digest_v2", Digest), (0x70000008, "plk_dim3_v2", Dim3), (0x70000009, "plk_geometry_v2", Geometry),
    (0x7000000A, "plk_header_v2", Header), (0x7000000B, "plk_layout_entry_v2", LayoutEntry),
    (0x7000000C, "plk_profile_digest_v2", ProfileDigest), (0x7000000D, "plk_resources_v2", Resources),
    (0x7000000E, "plk_scalar_v2", Scalar), (0x7000000F, "plk_shared_scalars_v2", SharedScalars),
    (0x70000010, "plk_transfer_report_v2", TransferReport), (0x70000011, "plk_tensor_meta_v2", TensorMeta),
    (0x70000012, "plk_workspace_demand_v2", WorkspaceDemand), (0x70000013, "plk_workspace_resource_v2", WorkspaceResource),
    (0x70000014, "plk_domain_v2", DomainRecord),
]

# ctypes mirrors of the owner-local record types a link may name (C name -> mirror)
MIRRORS = {"MokGemmResidue": MokGemmResidue, "MokActResidue": MokActResidue, "MokFrameworkParams": MokFrameworkParams,
           "MokMxView": MokMxView}
_TERM = re.compile(r"^(?:(\d+)|([A-Za-z_][\w.]*)|(floor|ceil)\(([A-Za-z_][\w.]*),(\d+)\))$")


def host_inventory(link: Mapping[str, Any]) -> dict[str, Any]:
    """link.json["host"], or the failure the reference's broker raises without one (broker.py:818-820)."""
    host = link.get("host")
    if not host or host.get("protocol") != 2:
        raise PlkError(4, "link.host: a link with a host section (protocol 2) is required")
    return host


def evaluate_extents(text: str, scalars: Mapping[str, Any]) -> tuple[int, ...]:
    """A channel's extents: comma-separated integers, scalar names, floor(name,int) or ceil(name,int)."""
    out = []
    for term in re.findall(r"(?:floor|ceil)\([^)]*\)|[^,]+", text.replace(" ", "")):
        m = _TERM.match(term)
        if not m:
            raise PlkError(4, f"link.host: cannot read the extent term {term!r}")
        if m.group(1):
            out.append(int(m.group(1)))
            continue
        name = m.group(2) or m.group(4)
        if name not in scalars:
            raise PlkError(3, f"scalar {name} is missing")
        value = int(scalars[name])
        out.append(value if m.group(2) else value // int(m.group(5)) if m.group(3) == "floor" else -(-value // int(m.group(5))))
    return tuple(out)


def channel_shapes(link: Mapping[str, Any], scalars: Mapping[str, Any]) -> dict[str, dict[str, tuple[int, int, tuple[int, ...]]]]:
    """owner -> channel name -> (element bits, access, extents) for the given scalars, channels in id order."""
    access = {"read": ACCESS_READ, "write": ACCESS_WRITE}
    return {g["owner"]: {c["name"]: (c["elem_bits"], access[c["access"]], evaluate_extents(c["extents"], scalars))
                         for c in sorted(g["channels"], key=lambda c: c["id"])}
            for g in host_inventory(link)["groups"]}


def layout_digest(name: str, mirror: type[Structure]) -> bytes:
    """SHA-256 of "type{member@offset+size;...}" -- what a provider reports as compiler_layout."""
    text = name + "{" + "".join(f"{m}@{getattr(mirror, m).offset}+{getattr(mirror, m).size};" for m, *_ in mirror._fields_) + "}"
    return hashlib.sha256(text.encode()).digest()


def _header(record: Structure) -> None:
    record.header = Header(ABI_V2, sizeof(record))


def _check(status: int, what: str) -> None:
    if status:
        names = {1: "PLK_E_VERSION", 2: "PLK_E_CAPACITY", 3: "PLK_E_ARGUMENT", 4: "PLK_E_CONTRACT", 5: "PLK_E_RESOURCE",
                 6: "PLK_E_BUILD", 7: "PLK_E_RELEASE"}
        raise PlkError(status, f"{what}: provider returned {names.get(status, status)}")


class _Scalars:
    """The shared scalar image: header, then plk_scalar_v2 records (device-safe: offsets, no pointers)."""

    def __init__(self, values: Mapping[str, Any], declared: list[Mapping[str, Any]]):
        ids = {d["name"]: d for d in declared}
        unknown = set(values) - set(ids)
        if unknown:
            raise PlkError(3, f"unknown scalars {sorted(unknown)}")
        recs = b""
        for name in sorted(values, key=lambda n: ids[n]["id"]):
            v = values[name]
            if ids[name]["kind"] == "f64":
                recs += struct.pack("<IIQ", ids[name]["id"], SCALAR_F64, struct.unpack("<Q", struct.pack("<d", float(v)))[0])
            else:
                recs += struct.pack("<IIq", ids[name]["id"], SCALAR_I64, int(v))
        head = SharedScalars(Header(ABI_V2, sizeof(SharedScalars)), sizeof(SharedScalars) + len(recs), len(values), sizeof(SharedScalars))
        self.buffer = ctypes.create_string_buffer(bytes(head) + recs, sizeof(SharedScalars) + len(recs))
        self.pointer = cast(self.buffer, POINTER(SharedScalars))


class Owner:
    """One params group: its provider's four entry points and the records exchanged with it."""

    def __init__(self, lib: ctypes.CDLL, group: Mapping[str, Any]):
        self.group, self.stage_id = group, group["owner"]
        self.local_types = []
        for t in group["provider"]["abi_types"]:
            mirror = MIRRORS.get(t["name"])
            if mirror is None or sizeof(mirror) != t["bytes"] or ctypes.alignment(mirror) != t["align"]:
                raise PlkError(1, f"{self.stage_id}: the link declares {t['name']} ({t['bytes']} bytes, align {t['align']}), "
                                  "which this broker does not mirror")
            self.local_types.append((t["id"], t["name"], mirror))
        symbols = group["provider"]["symbols"]
        try:
            self.abi, self.query, self.build, self.release = (getattr(lib, symbols[k]) for k in ("abi", "query", "build", "release"))
        except AttributeError as err:
            raise PlkError(4, f"{self.stage_id}: missing provider export: {err}") from None
        self.abi.argtypes, self.abi.restype = [POINTER(AbiReport)], ctypes.c_int
        self.query.argtypes, self.query.restype = [POINTER(Common), c_void_p, POINTER(Demands)], ctypes.c_int
        self.build.argtypes = [POINTER(Common), c_void_p, POINTER(Resources), c_void_p, c_size_t, POINTER(TransferReport),
                               c_uint32, POINTER(c_void_p)]
        self.build.restype = ctypes.c_int
        self.release.argtypes, self.release.restype = [c_void_p], ctypes.c_int
        self.session = c_void_p()
        self.built = False

    def report(self) -> AbiReport:
        """abi: every record type's size, alignment and layout digest must equal this side's mirror."""
        types = NEUTRAL_TYPES + self.local_types
        entries = (LayoutEntry * len(types))()
        for entry, (type_id, _, _) in zip(entries, types):
            entry.abi_type_id = type_id
        rep = AbiReport()
        _header(rep)
        rep.entry_capacity, rep.entries = len(types), entries
        _check(self.abi(byref(rep)), f"{self.stage_id}: abi")
        if rep.entry_count != len(types):
            raise PlkError(4, f"{self.stage_id}: abi reported {rep.entry_count} types, expected {len(types)}")
        for entry, (type_id, name, mirror) in zip(entries, types):
            if entry.bytes != sizeof(mirror) or entry.alignment_bytes != ctypes.alignment(mirror) or \
                    bytes(entry.compiler_layout.sha256) != layout_digest(name, mirror):
                raise PlkError(1, f"{self.stage_id}: layout of {name} differs between provider and broker")
        self._keep = entries
        return rep


class HostSession:
    """What open_host returns: the params image on the device and a launch method (broker.py:741-801)."""

    def __init__(self, backend: Any):
        self.backend = backend
        self.owners: list[Owner] = []
        self.params_addr = 0
        self.image = b""
        self.geometry: dict[str, Any] = {}
        self.function = None
        self.module = None

    def launch(self, stream: int | None = None) -> None:
        g = self.geometry
        self.backend.launch(self.function, self.params_addr, g["grid"], g["block"], g["dyn_lds"], stream)

    def close(self) -> None:
        errors = []
        for owner in reversed(self.owners):  # reverse build order, before anything is freed
            if owner.built:
                status = owner.release(owner.session)
                owner.built = False
                if status:
                    errors.append(f"{owner.stage_id}: release returned {status}")
        if self.params_addr:
            self.backend.free(self.params_addr)
            self.params_addr = 0
        if self.module is not None:
            self.backend.module_unload(self.module)
            self.module = None
        if errors:
            raise PlkError(7, "; ".join(errors))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def plan(link: Mapping[str, Any], resources: Mapping[str, Mapping[str, Resource]], scalars: Mapping[str, Any], *,
         compute_units: int, lib: ctypes.CDLL | None = None, stream_token: int = 0,
         providers: Mapping[str, ctypes.CDLL] | None = None) -> tuple[bytes, dict[str, Any], list[Owner]]:
    """report -> query -> build for every owner; returns (params image, launch geometry, owners).

    Host-only: touches no device memory.  ``resources`` maps stage id -> channel name -> Resource."""
    host = host_inventory(link)
    groups = {g["owner"]: g for g in host["groups"]}
    if providers is not None:  # one library per params group, as the reference's open_host takes them (broker.py:824-827)
        if set(providers) != {g["params_group"] for g in host["groups"]}:
            raise PlkError(4, "providers must exactly resolve the link's params groups: "
                              f"expected {sorted(g['params_group'] for g in host['groups'])}, got {sorted(providers)}")
    else:
        lib = lib or load_library()
    entries = {e["stage_id"]: e for e in link["params"]["entries"]}
    blobs = {b["stage_id"] for b in host["params"]["blobs"] if b["bytes"]}
    if set(entries) - blobs != set(groups) or set(resources) != set(groups):
        raise PlkError(4, "link.json params entries and resources must name exactly the link's owners")
    missing = {d["name"] for d in host["scalars"]} - set(scalars)
    if missing:
        raise PlkError(3, f"scalars {sorted(missing)} are missing")
    shapes = channel_shapes(link, scalars)
    optional = {(g["owner"], c["name"]) for g in host["groups"] for c in g["channels"] if c["optional"]}
    shared = _Scalars(scalars, host["scalars"])
    block = Dim3(link["threads"], 1, 1)
    image = bytearray(link["params"]["total_bytes"])
    geometry: dict[str, Any] = {}
    owners: list[Owner] = []
    keep: list[Any] = [shared]
    try:
        for stage_id in (s["stage_id"] for s in link["params"]["entries"] if s["stage_id"] in groups):
            owner = Owner(providers[groups[stage_id]["params_group"]] if providers is not None else lib, groups[stage_id])
            owners.append(owner)
            rep = owner.report()
            names = list(shapes[stage_id])
            if set(resources[stage_id]) - set(names) or \
                    {n for n in names if (stage_id, n) not in optional} - set(resources[stage_id]):
                raise PlkError(4, f"{stage_id}: resources must cover channels {names}")
            n = len(names)
            metas, demands = (TensorMeta * n)(), (ChannelDemand * n)()
            for idx, name in enumerate(names):
                bits, access, extents = shapes[stage_id][name]
                present = name in resources[stage_id]
                if not present:
                    extents = tuple(0 for _ in extents)
                ext = (c_uint64 * len(extents))(*extents)
                strides, stride = [0] * len(extents), (bits if present and all(extents) else 0)
                for k in reversed(range(len(extents))):
                    strides[k] = stride
                    stride *= extents[k]
                st = (c_int64 * len(extents))(*strides)
                res = resources[stage_id].get(name, Resource(0, 0))
                metas[idx] = TensorMeta(idx + 1, 0, len(extents), access, res.allocation_bytes, 16, res.origin_byte_offset, 0, 0,
                                        ext, st)
                dext, dst = (c_uint64 * len(extents))(), (c_int64 * len(extents))()
                demands[idx] = ChannelDemand(idx + 1, 0, len(extents), 0, 0, 0, dext, dst)
                keep += [ext, st, dext, dst]
            common = Common()
            _header(common)
            common.owner_id, common.channel_count, common.domain_count = len(owners), n, 0
            common.shared, common.channels = shared.pointer, metas
            common.block, common.cluster = block, Dim3(1, 1, 1)
            common.dynamic_smem_bytes = link["dyn_smem_bytes"]
            common.profile, common.owner_contract = rep.profile, rep.owner_contract
            dem = Demands()
            _header(dem)
            dem.channel_capacity, dem.channels = n, demands
            _check(owner.query(byref(common), None, byref(dem)), f"{stage_id}: query")
            devres = (DeviceResource * n)()
            for idx, name in enumerate(names):
                res = resources[stage_id].get(name, Resource(0, 0))
                need = demands[idx].minimum_allocation_bytes
                if name in resources[stage_id] and (need > res.allocation_bytes - res.origin_byte_offset or
                                                    (res.address + res.origin_byte_offset) % max(1, demands[idx].alignment_bytes)):
                    raise PlkError(5, f"{stage_id}.{name}: needs {need} bytes aligned to {demands[idx].alignment_bytes}")
                devres[idx] = DeviceResource(idx + 1, demands[idx].access, res.address, res.allocation_bytes,
                                             res.origin_byte_offset, 0, 0, None, 0)
            if dem.geometry.geometry_present:
                wgs = min(int(dem.geometry.grid.x), compute_units * int(link.get("workgroups_per_cu", 1)))
                geometry = {"grid": ((wgs + 7) // 8 * 8, 1, 1), "block": (dem.geometry.block.x, 1, 1),
                            "dyn_lds": int(dem.geometry.dynamic_smem_bytes)}
            r = Resources()
            _header(r)
            r.channel_count, r.channels, r.shared, r.cuda_stream_token = n, devres, shared.pointer, stream_token
            entry = entries[stage_id]
            residue = ctypes.create_string_buffer(entry["bytes"])
            _check(owner.build(byref(common), None, byref(r), residue, entry["bytes"], None, 0, byref(owner.session)),
                   f"{stage_id}: build")
            owner.built = True
            image[entry["offset"]:entry["offset"] + entry["bytes"]] = residue.raw
            keep += [metas, demands, devres]
    except Exception:
        for owner in reversed(owners):
            if owner.built:
                owner.release(owner.session)
        raise
    if not geometry:
        raise PlkError(4, "no owner stated the launch geometry")
    return bytes(image), geometry, owners


def open_host(link: Mapping[str, Any], image: bytes, resources: Mapping[str, Mapping[str, Resource]],
              scalars: Mapping[str, Any], backend: Any, providers: Mapping[str, ctypes.CDLL] | None = None) -> HostSession:
    """Load the code object, plan the params image through the providers, put it on the device."""
    session = HostSession(backend)
    session.module = backend.module_load(image)
    try:
        session.function = backend.module_function(session.module, link["kernel_symbol"], link["dyn_smem_bytes"])
        session.image, session.geometry, session.owners = plan(link, resources, scalars,
                                                               compute_units=backend.info().compute_units,
                                                               stream_token=backend.stream_token, providers=providers)
        session.params_addr = backend.allocate(len(session.image), 256)
        backend.upload(session.params_addr, session.image)
        backend.synchronize()
    except Exception:
        session.close()
        raise
    return session
