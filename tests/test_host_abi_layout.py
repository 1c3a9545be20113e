"""The 20 neutral records of the host ABI, pinned as literal numbers.

The records are a wire format shared with the reference's providers and broker
(pipec/src/pipec2/host/include/pipelink_host_abi_v2.h:60-184): a member that moves, or padding that
appears, breaks every provider built against the other header without any symbol changing.  The
numbers below were worked out by hand from the member lists under the LP64 rules (natural alignment,
8-byte pointers); the test compiles ``include/plk_host_abi_v2.h`` with gcc and compares what the
compiler lays out, then checks the broker's ctypes mirrors against the same numbers."""
import ctypes
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# record -> (bytes, alignment, {member: offset})
LAYOUT = {
    "plk_header_v2": (8, 4, {"abi_version": 0, "struct_bytes": 4}),
    "plk_digest_v2": (32, 1, {"sha256": 0}),
    "plk_profile_digest_v2": (32, 1, {"dtypes": 0}),
    "plk_dim3_v2": (12, 4, {"x": 0, "y": 4, "z": 8}),
    "plk_scalar_v2": (16, 8, {"scalar_id": 0, "scalar_type": 4, "value_bits": 8}),
    "plk_shared_scalars_v2": (24, 8, {"header": 0, "image_bytes": 8, "record_count": 16, "record_offset": 20}),
    "plk_tensor_meta_v2": (64, 8, {"channel_id": 0, "dtype_id": 4, "rank": 8, "access": 12, "allocation_bytes": 16,
                                   "alignment_bytes": 24, "origin_byte_offset": 32, "origin_bit_offset": 40, "reserved": 44,
                                   "extents": 48, "bit_strides": 56}),
    "plk_geometry_v2": (56, 8, {"geometry_present": 0, "launch_required": 4, "grid": 8, "block": 20, "cluster": 32,
                                "reserved": 44, "dynamic_smem_bytes": 48}),
    "plk_domain_v2": (16, 4, {"domain_id": 0, "rank": 4, "world": 8, "reserved": 12}),
    "plk_common_v2": (144, 8, {"header": 0, "owner_id": 8, "channel_count": 12, "domain_count": 16, "reserved": 20, "shared": 24,
                               "channels": 32, "domains": 40, "block": 48, "cluster": 60, "dynamic_smem_bytes": 72,
                               "profile": 80, "owner_contract": 112}),
    "plk_channel_demand_v2": (48, 8, {"channel_id": 0, "dtype_id": 4, "rank": 8, "access": 12, "minimum_allocation_bytes": 16,
                                      "alignment_bytes": 24, "extents": 32, "bit_strides": 40}),
    "plk_workspace_demand_v2": (24, 8, {"workspace_id": 0, "reserved": 4, "bytes": 8, "alignment_bytes": 16}),
    "plk_demands_v2": (96, 8, {"header": 0, "channel_count": 8, "channel_capacity": 12, "channels": 16, "workspace_count": 24,
                               "workspace_capacity": 28, "workspaces": 32, "geometry": 40}),
    "plk_device_resource_v2": (56, 8, {"channel_id": 0, "access": 4, "allocation_address": 8, "allocation_bytes": 16,
                                       "origin_byte_offset": 24, "origin_bit_offset": 32, "domain_id": 36, "peer_addresses": 40,
                                       "multicast_address": 48}),
    "plk_workspace_resource_v2": (32, 8, {"workspace_id": 0, "reserved": 4, "device_address": 8, "bytes": 16, "alignment_bytes": 24}),
    "plk_resources_v2": (104, 8, {"header": 0, "channel_count": 8, "workspace_count": 12, "channels": 16, "workspaces": 24,
                                  "shared": 32, "cuda_stream_token": 40, "geometry": 48}),
    "plk_tma_tiled_detail_v2": (72, 8, {"swizzle": 0, "rank": 4, "box_elements": 8, "element_strides": 48, "reserved": 68}),
    "plk_transfer_report_v2": (96, 8, {"transfer_id": 0, "access": 4, "residue_offset": 8, "representation_bytes": 16,
                                       "representation_align": 24, "storage_dtype_id": 32, "ring_depth": 36,
                                       "ring_stage_stride_bytes": 40, "footprint_bytes_per_stage": 48, "credit_bytes_per_stage": 56,
                                       "source_origin_bits": 64, "source_span_bits": 72, "vendor_kind": 80, "reserved": 84,
                                       "vendor_detail": 88}),
    "plk_layout_entry_v2": (56, 8, {"abi_type_id": 0, "reserved": 4, "bytes": 8, "alignment_bytes": 16, "compiler_layout": 24}),
    "plk_abi_report_v2": (88, 8, {"header": 0, "entry_count": 8, "entry_capacity": 12, "entries": 16, "profile": 24,
                                  "owner_contract": 56}),
}


@pytest.mark.skipif(shutil.which("gcc") is None, reason="needs gcc")
def test_the_header_lays_the_records_out_as_pinned(tmp_path):
    assert len(LAYOUT) == 20
    lines = ['#include <stdio.h>', '#include <stddef.h>', '#include "plk_host_abi_v2.h"', "int main(void) {"]
    for name, (_, _, members) in LAYOUT.items():
        lines.append(f'  printf("{name} %zu %zu", sizeof({name}), _Alignof({name}));')
        for m in members:
            lines.append(f'  printf(" {m}=%zu", offsetof({name}, {m}));')
        lines.append('  printf("\\n");')
    lines += [f'  printf("count %u\\n", (unsigned)PLK_ABI_NEUTRAL_TYPE_COUNT);', "  return 0;", "}"]
    src = tmp_path / "layout.c"
    src.write_text("\n".join(lines))
    exe = tmp_path / "layout"
    subprocess.run(["gcc", "-std=c11", "-Wall", "-Werror", f"-I{os.path.join(ROOT, 'include')}", str(src), "-o", str(exe)], check=True)
    seen = {}
    for line in subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.splitlines():
        name, *rest = line.split()
        if name == "count":
            assert rest == ["20"]
            continue
        seen[name] = (int(rest[0]), int(rest[1]), {m: int(o) for m, o in (kv.split("=") for kv in rest[2:])})
    assert seen == LAYOUT


def test_the_brokers_mirrors_have_the_pinned_sizes():
    from pipelink_amd.host import broker

    mirrors = {"plk_header_v2": "Header", "plk_digest_v2": "Digest", "plk_profile_digest_v2": "ProfileDigest", "plk_domain_v2": "DomainRecord",
               "plk_tma_tiled_detail_v2": "TmaTiledDetail", "plk_dim3_v2": "Dim3", "plk_scalar_v2": "Scalar",
               "plk_shared_scalars_v2": "SharedScalars", "plk_tensor_meta_v2": "TensorMeta", "plk_geometry_v2": "Geometry",
               "plk_common_v2": "Common", "plk_channel_demand_v2": "ChannelDemand", "plk_workspace_demand_v2": "WorkspaceDemand",
               "plk_demands_v2": "Demands", "plk_device_resource_v2": "DeviceResource",
               "plk_workspace_resource_v2": "WorkspaceResource", "plk_resources_v2": "Resources",
               "plk_transfer_report_v2": "TransferReport", "plk_layout_entry_v2": "LayoutEntry", "plk_abi_report_v2": "AbiReport"}
    checked = 0
    for record, cls_name in mirrors.items():
        cls = getattr(broker, cls_name)
        size, align, members = LAYOUT[record]
        assert (ctypes.sizeof(cls), ctypes.alignment(cls)) == (size, align), record
        for m, off in members.items():
            if hasattr(cls, m):
                assert getattr(cls, m).offset == off, (record, m)
        checked += 1
    assert checked == 20
