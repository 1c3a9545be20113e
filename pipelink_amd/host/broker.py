"""Broker side of the PipeLink host ABI v2: report / query / build each owner once, assemble the
params image at the linked offsets, launch.

Plays the part of ``pipec2.host.broker.open_host`` (pipec/src/pipec2/host/broker.py:804-949) for
the routed-expert FFN pipeline: the owners' providers (``pipelink_params_{abi,query,build,
release}_<suffix>``, include/plk_host_abi_v2.h) live in the C-ABI library; the broker owns every
record, array and the residue bytes, checks each provider's answers against what the caller
holds, and releases sessions in reverse build order (broker.py:768-801).  What the reference
reads from the ``host`` section of link.json (owner inventory, channel lists) is the table
``OWNERS`` here -- the three owners and their channels are fixed for this pipeline.

Pure ctypes; nothing here needs a GPU until ``HostSession.launch``."""
from __future__ import annotations

import ctypes
import hashlib
import struct
from ctypes import (POINTER, Structure, byref, c_int64, c_size_t, c_uint8, c_uint32, c_uint64, c_void_p, cast, pointer,
                    sizeof)
from dataclasses import dataclass
from typing import Any, Mapping

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


class Domain(Structure):
    _fields_ = [("domain_id", c_uint32), ("rank", c_uint32), ("world", c_uint32), ("reserved", c_uint32)]


class Common(Structure):
    _fields_ = [("header", Header), ("owner_id", c_uint32), ("channel_count", c_uint32), ("domain_count", c_uint32),
                ("reserved", c_uint32), ("shared", POINTER(SharedScalars)), ("channels", POINTER(TensorMeta)),
                ("domains", POINTER(Domain)), ("block", Dim3), ("cluster", Dim3), ("dynamic_smem_bytes", c_uint64),
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
    _fields_ = [("tokens_per_expert", c_void_p), ("expert_row_begin", c_void_p), ("expert_tile_begin", c_void_p),
                ("num_experts", ctypes.c_int32), ("op", ctypes.c_int32), ("num_col_tiles", ctypes.c_int32),
                ("reserved", ctypes.c_int32)]


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
    (0x70000014, "plk_domain_v2", Domain),
]

# scalar ids (include/plk_host_abi_v2.h)
SCALARS = {"mok.num_local_tokens": 1, "mok.hidden": 2, "mok.intermediate": 3, "mok.num_local_experts": 4,
           "mok.swiglu_limit": 10, "mok.pass": 11, "mok.precision": 12, "mok.routed_rows": 60, "mok.ld_q_h": 61,
           "mok.ld_q_i": 62, "mok.ld_sc_h": 63, "mok.ld_sc_i": 64}


def _shapes(s: Mapping[str, int]) -> dict[str, dict[str, tuple[int, int, tuple[int, ...]]]]:
    """(element bits, access, extents) of every channel of every owner for the given scalars."""
    t, h, i, e, r = (s[k] for k in ("mok.num_local_tokens", "mok.hidden", "mok.intermediate", "mok.num_local_experts",
                                    "mok.routed_rows"))
    wq = lambda n, k: (8, ACCESS_READ, (e, k // 64, n, 64))
    wsc = lambda n, k: (8, ACCESS_READ, (e, (k + 127) // 128, n, 4))
    return {
        "mok.framework": {"tokens_per_expert": (32, ACCESS_READ, (e,))},
        "mok.gemm": {
            "x_q": (8, ACCESS_READ, (t, s["mok.ld_q_h"])), "x_sc": (8, ACCESS_READ, (t, s["mok.ld_sc_h"])),
            "w_gate_q": wq(i, h), "w_gate_sc": wsc(i, h), "w_up_q": wq(i, h), "w_up_sc": wsc(i, h),
            "w_down_q": wq(h, i), "w_down_sc": wsc(h, i),
            "hidden_q": (8, ACCESS_READ, (r, s["mok.ld_q_i"])), "hidden_sc": (8, ACCESS_READ, (r, s["mok.ld_sc_i"])),
            "y": (16, ACCESS_WRITE, (r, h)), "row_token": (32, ACCESS_READ, (r,)),
        },
        "mok.act": {"hidden_q": (8, ACCESS_WRITE, (r, s["mok.ld_q_i"])), "hidden_sc": (8, ACCESS_WRITE, (r, s["mok.ld_sc_i"]))},
    }


# stage id -> (entry point suffix, owner-local types it reports: (id, C name, mirror))
OWNERS = {
    "mok.framework": ("mok_framework", [(3, "MokFrameworkParams", MokFrameworkParams)]),
    "mok.gemm": ("mok_gemm", [(1, "MokGemmResidue", MokGemmResidue), (4, "MokMxView", MokMxView)]),
    "mok.act": ("mok_act", [(2, "MokActResidue", MokActResidue)]),
}
OPTIONAL = {("mok.gemm", "row_token")}


def layout_digest(name: str, mirror: type[Structure]) -> bytes:
    """SHA-256 of "type{member@offset+size;...}" -- what a provider reports as compiler_layout."""
    text = name + "{" + "".join(f"{m}@{getattr(mirror, m).offset}+{getattr(mirror, m).size};" for m, *_ in mirror._fields_) + "}"
    return hashlib.sha256(text.encode()).digest()


@dataclass
class Resource:
    """One caller-owned device allocation (host/fixture.py:22-40 in the reference)."""
    address: int
    allocation_bytes: int
    origin_byte_offset: int = 0


def _header(record: Structure) -> None:
    record.header = Header(ABI_V2, sizeof(record))


def _check(status: int, what: str) -> None:
    if status:
        names = {1: "PLK_E_VERSION", 2: "PLK_E_CAPACITY", 3: "PLK_E_ARGUMENT", 4: "PLK_E_CONTRACT", 5: "PLK_E_RESOURCE",
                 6: "PLK_E_BUILD", 7: "PLK_E_RELEASE"}
        raise PlkError(status, f"{what}: provider returned {names.get(status, status)}")


class _Scalars:
    """The shared scalar image: header, then plk_scalar_v2 records (device-safe: offsets, no pointers)."""

    def __init__(self, values: Mapping[str, Any]):
        unknown = set(values) - set(SCALARS)
        if unknown:
            raise PlkError(3, f"unknown scalars {sorted(unknown)}")
        recs = b""
        for name in sorted(values, key=SCALARS.get):
            v = values[name]
            if name == "mok.swiglu_limit":
                recs += struct.pack("<IIQ", SCALARS[name], SCALAR_F64, struct.unpack("<Q", struct.pack("<d", float(v)))[0])
            else:
                recs += struct.pack("<IIq", SCALARS[name], SCALAR_I64, int(v))
        head = SharedScalars(Header(ABI_V2, sizeof(SharedScalars)), sizeof(SharedScalars) + len(recs), len(values), sizeof(SharedScalars))
        self.buffer = ctypes.create_string_buffer(bytes(head) + recs, sizeof(SharedScalars) + len(recs))
        self.pointer = cast(self.buffer, POINTER(SharedScalars))


class Owner:
    """One params group: its provider's four entry points and the records exchanged with it."""

    def __init__(self, lib: ctypes.CDLL, stage_id: str):
        self.stage_id = stage_id
        suffix, self.local_types = OWNERS[stage_id]
        self.abi = getattr(lib, f"pipelink_params_abi_{suffix}")
        self.query = getattr(lib, f"pipelink_params_query_{suffix}")
        self.build = getattr(lib, f"pipelink_params_build_{suffix}")
        self.release = getattr(lib, f"pipelink_params_release_{suffix}")
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
         compute_units: int, lib: ctypes.CDLL | None = None, stream_token: int = 0) -> tuple[bytes, dict[str, Any], list[Owner]]:
    """report -> query -> build for every owner; returns (params image, launch geometry, owners).

    Host-only: touches no device memory.  ``resources`` maps stage id -> channel name -> Resource."""
    lib = lib or load_library()
    entries = {e["stage_id"]: e for e in link["params"]["entries"]}
    if set(entries) != set(OWNERS) or set(resources) != set(OWNERS):
        raise PlkError(4, "link.json params entries and resources must name exactly the pipeline's owners")
    missing = set(SCALARS) - set(scalars)
    if missing:
        raise PlkError(3, f"scalars {sorted(missing)} are missing")
    shapes = _shapes(scalars)
    shared = _Scalars(scalars)
    block = Dim3(link["threads"], 1, 1)
    image = bytearray(link["params"]["total_bytes"])
    geometry: dict[str, Any] = {}
    owners: list[Owner] = []
    keep: list[Any] = [shared]
    try:
        for stage_id in (s["stage_id"] for s in link["params"]["entries"]):
            owner = Owner(lib, stage_id)
            owners.append(owner)
            rep = owner.report()
            names = list(shapes[stage_id])
            if set(resources[stage_id]) - set(names) or \
                    {n for n in names if (stage_id, n) not in OPTIONAL} - set(resources[stage_id]):
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
              scalars: Mapping[str, Any], backend: Any) -> HostSession:
    """Load the code object, plan the params image through the providers, put it on the device."""
    session = HostSession(backend)
    session.module = backend.module_load(image)
    try:
        session.function = backend.module_function(session.module, link["kernel_symbol"], link["dyn_smem_bytes"])
        session.image, session.geometry, session.owners = plan(link, resources, scalars,
                                                               compute_units=backend.info().compute_units,
                                                               stream_token=backend.stream_token)
        session.params_addr = backend.allocate(len(session.image), 256)
        backend.upload(session.params_addr, session.image)
        backend.synchronize()
    except Exception:
        session.close()
        raise
    return session
