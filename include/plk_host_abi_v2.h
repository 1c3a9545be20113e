/* PipeLink host ABI v2 as the MI355X build speaks it: the record types a broker and an owner's
 * provider exchange, and the four entry points every owner of the routed-expert FFN exports.
 *
 * Binary interface of the reference's pipec/src/pipec2/host/include/pipelink_host_abi_v2.h
 * (type names, member names, member order and the neutral type IDs at :255-275 are the wire
 * format; a provider built against either header loads into either broker).  What differs
 * here is on the far side of the records: `cuda_stream_token` carries a hipStream_t, device
 * addresses are HIP device addresses, and the only transfer kind an owner reports is
 * PLK_TRANSFER_STRIDED -- gfx950 has no tensor-map encoder, an owner's residue holds plain
 * {address, rows, k, pitch} views.
 *
 * Calling rules (reference: host/broker.py:768-949, host ABI header :1-12,21-28,43-47):
 *   - every record that starts with plk_header_v2 is checked: abi_version == 2 and
 *     struct_bytes == sizeof(record), else PLK_E_VERSION;
 *   - the caller owns every array and the residue bytes and states capacities; the provider
 *     fills them and never keeps a pointer past the call;
 *   - `build` hands back at most one opaque session per success; `release` takes it exactly
 *     once (a null session is fine), in reverse build order, before the caller frees anything;
 *   - no exception, enum, bitfield or packed record crosses; status codes below;
 *   - single-threaded, device current on the calling thread, no provider global state. */
#ifndef PLK_HOST_ABI_V2_H
#define PLK_HOST_ABI_V2_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PLK_HOST_ABI_V2 2u

/* status codes (shared with plk_hip.h) */
#ifndef PLK_STATUS_CODES_DEFINED
#define PLK_STATUS_CODES_DEFINED
enum {
  PLK_OK = 0,
  PLK_E_VERSION = 1,
  PLK_E_CAPACITY = 2,
  PLK_E_ARGUMENT = 3,
  PLK_E_CONTRACT = 4,
  PLK_E_RESOURCE = 5,
  PLK_E_BUILD = 6,
  PLK_E_RELEASE = 7
};
#endif

#define PLK_SCALAR_U64 1u
#define PLK_SCALAR_I64 2u
#define PLK_SCALAR_F64 3u
#define PLK_SCALAR_BOOL 4u

#define PLK_ACCESS_READ 1u
#define PLK_ACCESS_WRITE 2u
#define PLK_ACCESS_READ_WRITE 3u

#define PLK_TRANSFER_TMA_TILED 1u  /* never reported by a gfx950 owner */
#define PLK_TRANSFER_TMA_IM2COL 2u /* never reported by a gfx950 owner */
#define PLK_TRANSFER_STRIDED 3u

typedef struct plk_header_v2 { uint32_t abi_version, struct_bytes; } plk_header_v2;
typedef struct plk_digest_v2 { uint8_t sha256[32]; } plk_digest_v2;
typedef struct plk_profile_digest_v2 { plk_digest_v2 dtypes; } plk_profile_digest_v2;
typedef struct plk_dim3_v2 { uint32_t x, y, z; } plk_dim3_v2;
typedef struct plk_scalar_v2 { uint32_t scalar_id, scalar_type; uint64_t value_bits; } plk_scalar_v2;

/* scalar image shared by all owners of a session: record_offset is relative to the header */
typedef struct plk_shared_scalars_v2 {
  plk_header_v2 header;
  uint64_t image_bytes;
  uint32_t record_count, record_offset;
} plk_shared_scalars_v2;

/* what the caller says about one tensor at query time (no addresses yet) */
typedef struct plk_tensor_meta_v2 {
  uint32_t channel_id, dtype_id, rank, access;
  uint64_t allocation_bytes, alignment_bytes, origin_byte_offset;
  uint32_t origin_bit_offset, reserved;
  const uint64_t* extents;
  const int64_t* bit_strides;
} plk_tensor_meta_v2;

typedef struct plk_geometry_v2 {
  uint32_t geometry_present, launch_required;
  plk_dim3_v2 grid, block, cluster;
  uint32_t reserved;
  uint64_t dynamic_smem_bytes;
} plk_geometry_v2;

typedef struct plk_domain_v2 { uint32_t domain_id, rank, world, reserved; } plk_domain_v2;

typedef struct plk_common_v2 {
  plk_header_v2 header;
  uint32_t owner_id, channel_count, domain_count, reserved;
  const plk_shared_scalars_v2* shared;
  const plk_tensor_meta_v2* channels;
  const plk_domain_v2* domains;
  plk_dim3_v2 block, cluster;
  uint64_t dynamic_smem_bytes;
  plk_profile_digest_v2 profile;
  plk_digest_v2 owner_contract;
} plk_common_v2;

/* the owner's answer at query time; ids, ranks, array pointers and capacities come pre-filled */
typedef struct plk_channel_demand_v2 {
  uint32_t channel_id, dtype_id, rank, access;
  uint64_t minimum_allocation_bytes, alignment_bytes;
  uint64_t* extents;
  int64_t* bit_strides;
} plk_channel_demand_v2;
typedef struct plk_workspace_demand_v2 { uint32_t workspace_id, reserved; uint64_t bytes, alignment_bytes; } plk_workspace_demand_v2;
typedef struct plk_demands_v2 {
  plk_header_v2 header;
  uint32_t channel_count, channel_capacity;
  plk_channel_demand_v2* channels;
  uint32_t workspace_count, workspace_capacity;
  plk_workspace_demand_v2* workspaces;
  plk_geometry_v2 geometry;
} plk_demands_v2;

/* what the caller hands to build: bounded device allocations (one GPU: no peer views) */
typedef struct plk_device_resource_v2 {
  uint32_t channel_id, access;
  uint64_t allocation_address, allocation_bytes, origin_byte_offset;
  uint32_t origin_bit_offset, domain_id;
  const uint64_t* peer_addresses;
  uint64_t multicast_address;
} plk_device_resource_v2;
typedef struct plk_workspace_resource_v2 { uint32_t workspace_id, reserved; uint64_t device_address, bytes, alignment_bytes; } plk_workspace_resource_v2;
typedef struct plk_resources_v2 {
  plk_header_v2 header;
  uint32_t channel_count, workspace_count;
  const plk_device_resource_v2* channels;
  const plk_workspace_resource_v2* workspaces;
  const plk_shared_scalars_v2* shared;
  uint64_t cuda_stream_token; /* a hipStream_t here */
  plk_geometry_v2 geometry;
} plk_resources_v2;

typedef struct plk_tma_tiled_detail_v2 {
  uint32_t swizzle, rank;
  uint64_t box_elements[5];
  uint32_t element_strides[5];
  uint32_t reserved;
} plk_tma_tiled_detail_v2;

/* one per declared transfer, filled by build */
typedef struct plk_transfer_report_v2 {
  uint32_t transfer_id, access;
  uint64_t residue_offset, representation_bytes, representation_align;
  uint32_t storage_dtype_id, ring_depth;
  uint64_t ring_stage_stride_bytes, footprint_bytes_per_stage, credit_bytes_per_stage;
  uint64_t source_origin_bits, source_span_bits;
  uint32_t vendor_kind, reserved;
  const void* vendor_detail;
} plk_transfer_report_v2;

typedef struct plk_layout_entry_v2 {
  uint32_t abi_type_id, reserved;
  uint64_t bytes, alignment_bytes;
  plk_digest_v2 compiler_layout;
} plk_layout_entry_v2;
typedef struct plk_abi_report_v2 {
  plk_header_v2 header;
  uint32_t entry_count, entry_capacity;
  plk_layout_entry_v2* entries;
  plk_profile_digest_v2 profile;
  plk_digest_v2 owner_contract;
} plk_abi_report_v2;

/* neutral type ids (wire values of the reference header's inventory) */
#define PLK_ABI_TYPE_ID_plk_abi_report_v2 0x70000001u
#define PLK_ABI_TYPE_ID_plk_channel_demand_v2 0x70000002u
#define PLK_ABI_TYPE_ID_plk_common_v2 0x70000003u
#define PLK_ABI_TYPE_ID_plk_demands_v2 0x70000004u
#define PLK_ABI_TYPE_ID_plk_tma_tiled_detail_v2 0x70000005u
#define PLK_ABI_TYPE_ID_plk_device_resource_v2 0x70000006u
#define PLK_ABI_TYPE_ID_plk_digest_v2 0x70000007u
#define PLK_ABI_TYPE_ID_plk_dim3_v2 0x70000008u
#define PLK_ABI_TYPE_ID_plk_geometry_v2 0x70000009u
#define PLK_ABI_TYPE_ID_plk_header_v2 0x7000000au
#define PLK_ABI_TYPE_ID_plk_layout_entry_v2 0x7000000bu
#define PLK_ABI_TYPE_ID_plk_profile_digest_v2 0x7000000cu
#define PLK_ABI_TYPE_ID_plk_resources_v2 0x7000000du
#define PLK_ABI_TYPE_ID_plk_scalar_v2 0x7000000eu
#define PLK_ABI_TYPE_ID_plk_shared_scalars_v2 0x7000000fu
#define PLK_ABI_TYPE_ID_plk_transfer_report_v2 0x70000010u
#define PLK_ABI_TYPE_ID_plk_tensor_meta_v2 0x70000011u
#define PLK_ABI_TYPE_ID_plk_workspace_demand_v2 0x70000012u
#define PLK_ABI_TYPE_ID_plk_workspace_resource_v2 0x70000013u
#define PLK_ABI_TYPE_ID_plk_domain_v2 0x70000014u
#define PLK_ABI_NEUTRAL_TYPE_COUNT 20u

typedef struct plk_session_v2 plk_session; /* provider-owned, opaque */

/* ---- the routed-expert FFN owners -----------------------------------------------------------
 * Owner-local type ids (the residue records of pipelink_amd/stages/mok/include/mok_abi.h): */
#define MOK_ABI_TYPE_ID_MokGemmResidue 1u
#define MOK_ABI_TYPE_ID_MokActResidue 2u
#define MOK_ABI_TYPE_ID_MokFrameworkParams 3u
#define MOK_ABI_TYPE_ID_MokMxView 4u

/* Shared scalars the owners read (ids of campaigns/mok/port/include/mok_abi.h:57-70 where the
 * meaning is the same; the pitches have no counterpart there).  All PLK_SCALAR_I64 except the
 * limit, which is PLK_SCALAR_F64. */
#define MOK_SCALAR_NUM_LOCAL_TOKENS 1u   /* T */
#define MOK_SCALAR_HIDDEN 2u             /* H = d_model */
#define MOK_SCALAR_INTERMEDIATE 3u       /* I = d_ff */
#define MOK_SCALAR_NUM_LOCAL_EXPERTS 4u  /* E */
#define MOK_SCALAR_SWIGLU_LIMIT 10u      /* f64 */
#define MOK_SCALAR_PASS 11u              /* 0 = both GEMMs in one launch, 1 = gate/up + SwiGLU + requant, 2 = down */
#define MOK_SCALAR_PRECISION 12u         /* 1 = MXFP8 (the only one built) */
#define MOK_SCALAR_ROUTED_ROWS 60u       /* R = sum(tokens_per_expert) */
#define MOK_SCALAR_LD_Q_H 61u            /* code row pitch of x, bytes */
#define MOK_SCALAR_LD_Q_I 62u            /* code row pitch of hidden, bytes */
#define MOK_SCALAR_LD_SC_H 63u           /* scale row pitch of x */
#define MOK_SCALAR_LD_SC_I 64u           /* scale row pitch of hidden */
#define MOK_SCALAR_WORKSPACE_WORDS 65u   /* 32 + ceil(R / 256) + E: words of the launch workspace */

/* Channels of owner mok.gemm (channel_id = index + 1), all u8 unless noted:
 *   1 x_q [T, ld_q_h] R          2 x_sc [T, ld_sc_h] R
 *   3 w_gate_q [E, H/64, I, 64] R   4 w_gate_sc [E, ceil(H/128), I, 4] R
 *   5 w_up_q   (as 3) R             6 w_up_sc   (as 4) R
 *   7 w_down_q [E, I/64, H, 64] R   8 w_down_sc [E, ceil(I/128), H, 4] R
 *   9 hidden_q [R, ld_q_i] R       10 hidden_sc [R, ld_sc_i] R
 *  11 y [R, H] bf16 W              12 row_token [R] i32 R (a zero-size resource = rows are tokens)
 * Channels of owner mok.act:       1 hidden_q [R, ld_q_i] W   2 hidden_sc [R, ld_sc_i] W
 * Channels of owner mok.framework: 1 tokens_per_expert [E] i32 R
 *                                  2 workspace [workspace_words] u32 W: status word and readiness counters of a launch;
 *                                    all zero before the first launch, every launch leaves it zero again (but for
 *                                    word 0, the sticky status: bit 0 = a bounded dependency wait gave up) */
#define MOK_GEMM_CHANNEL_COUNT 12u
#define MOK_ACT_CHANNEL_COUNT 2u
#define MOK_FRAMEWORK_CHANNEL_COUNT 2u

/* Entry points, one set per owner suffix (reference: host ABI header :293-300 and
 * campaigns/mok/port/gemm/provider.cu:217-303).  `args` must be null: everything an owner
 * needs arrives as shared scalars and channels.
 *   abi     : caller pre-fills entries[i].abi_type_id and entry_capacity; the provider writes
 *             size, alignment and a SHA-256 of "type{member@offset+size;...}" for each.
 *   query   : checks block = 256x1x1, cluster 1x1x1, scalars, each channel's rank / access /
 *             extents / dense bit strides; writes minimum bytes and alignment per channel and,
 *             for mok.framework, the launch geometry (grid, block, dynamic LDS).
 *   build   : checks every resource against the demand and writes the owner's residue into
 *             `residue` (capacity `residue_cap`); transfer_capacity must be 0.
 *   release : null session only (no owner keeps host state). */
#define PLK_DECLARE_OWNER(suffix)                                                                          \
  int pipelink_params_abi_##suffix(plk_abi_report_v2* out);                                                \
  int pipelink_params_query_##suffix(const plk_common_v2* common, const void* args, plk_demands_v2* out);  \
  int pipelink_params_build_##suffix(const plk_common_v2* common, const void* args,                        \
                                     const plk_resources_v2* resources, void* residue, size_t residue_cap, \
                                     plk_transfer_report_v2* transfers, uint32_t transfer_capacity,       \
                                     plk_session** session);                                               \
  int pipelink_params_release_##suffix(plk_session* session);
PLK_DECLARE_OWNER(mok_gemm)
PLK_DECLARE_OWNER(mok_act)
PLK_DECLARE_OWNER(mok_framework)

#ifdef __cplusplus
}
#endif
#endif
