// Provider side of the PipeLink host ABI v2 for the three owners of the routed-expert FFN
// pipeline (mok.framework, mok.gemm, mok.act): abi / query / build / release, as declared in
// include/plk_host_abi_v2.h.  Plays the part of campaigns/mok/port/gemm/provider.cu:217-303
// (and its act / framework siblings) in the reference; the residues it writes are the plain
// {address, rows, k, pitch} views of pipelink_amd/stages/mok/include/mok_abi.h -- there is no
// descriptor encoder on gfx950.  Pure host code: nothing here touches the device.
#include <cstring>
#include <string>

#include "plk_host_abi_v2.h"
#include "plk_mok_residues.hpp"

namespace {

// ---- SHA-256 (FIPS 180-4) for the layout digests --------------------------------------------
struct Sha256 {
  uint32_t h[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
  static uint32_t rotr(uint32_t x, int n) { return (x >> n) | (x << (32 - n)); }
  void block(const unsigned char* p) {
    static const uint32_t k[64] = {
        0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01,
        0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174, 0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc,
        0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147,
        0x06ca6351, 0x14292967, 0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85,
        0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070, 0x19a4c116, 0x1e376c08,
        0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208,
        0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
    uint32_t w[64];
    for (int i = 0; i < 16; ++i) w[i] = (uint32_t)p[4 * i] << 24 | (uint32_t)p[4 * i + 1] << 16 | (uint32_t)p[4 * i + 2] << 8 | p[4 * i + 3];
    for (int i = 16; i < 64; ++i) {
      const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
      const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
      w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = h[0], b = h[1], c = h[2], d = h[3], e = h[4], f = h[5], g = h[6], hh = h[7];
    for (int i = 0; i < 64; ++i) {
      const uint32_t t1 = hh + (rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25)) + ((e & f) ^ (~e & g)) + k[i] + w[i];
      const uint32_t t2 = (rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22)) + ((a & b) ^ (a & c) ^ (b & c));
      hh = g; g = f; f = e; e = d + t1; d = c; c = b; b = a; a = t1 + t2;
    }
    h[0] += a; h[1] += b; h[2] += c; h[3] += d; h[4] += e; h[5] += f; h[6] += g; h[7] += hh;
  }
  static plk_digest_v2 of(const std::string& text) {
    Sha256 s;
    std::string m = text;
    const uint64_t bits = (uint64_t)text.size() * 8;
    m.push_back((char)0x80);
    while (m.size() % 64 != 56) m.push_back('\0');
    for (int i = 7; i >= 0; --i) m.push_back((char)(bits >> (8 * i)));
    for (size_t i = 0; i < m.size(); i += 64) s.block(reinterpret_cast<const unsigned char*>(m.data()) + i);
    plk_digest_v2 d;
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 4; ++j) d.sha256[4 * i + j] = (uint8_t)(s.h[i] >> (24 - 8 * j));
    return d;
  }
};

// ---- layout inventory: "type{member@offset+size;...}" ----------------------------------------
struct Layout {
  uint32_t id;
  uint64_t bytes, align;
  std::string text;
};
#define M(T, m) (std::string(#m) + "@" + std::to_string(offsetof(T, m)) + "+" + std::to_string(sizeof(((T*)0)->m)) + ";")
#define L(ID, T, ...) Layout{ID, sizeof(T), alignof(T), std::string(#T) + "{" + __VA_ARGS__ + "}"}

std::vector<Layout> inventory(const char* owner) {
  std::vector<Layout> v = {
      L(PLK_ABI_TYPE_ID_plk_abi_report_v2, plk_abi_report_v2, M(plk_abi_report_v2, header) + M(plk_abi_report_v2, entry_count) + M(plk_abi_report_v2, entry_capacity) + M(plk_abi_report_v2, entries) + M(plk_abi_report_v2, profile) + M(plk_abi_report_v2, owner_contract)),
      L(PLK_ABI_TYPE_ID_plk_channel_demand_v2, plk_channel_demand_v2, M(plk_channel_demand_v2, channel_id) + M(plk_channel_demand_v2, dtype_id) + M(plk_channel_demand_v2, rank) + M(plk_channel_demand_v2, access) + M(plk_channel_demand_v2, minimum_allocation_bytes) + M(plk_channel_demand_v2, alignment_bytes) + M(plk_channel_demand_v2, extents) + M(plk_channel_demand_v2, bit_strides)),
      L(PLK_ABI_TYPE_ID_plk_common_v2, plk_common_v2, M(plk_common_v2, header) + M(plk_common_v2, owner_id) + M(plk_common_v2, channel_count) + M(plk_common_v2, domain_count) + M(plk_common_v2, reserved) + M(plk_common_v2, shared) + M(plk_common_v2, channels) + M(plk_common_v2, domains) + M(plk_common_v2, block) + M(plk_common_v2, cluster) + M(plk_common_v2, dynamic_smem_bytes) + M(plk_common_v2, profile) + M(plk_common_v2, owner_contract)),
      L(PLK_ABI_TYPE_ID_plk_demands_v2, plk_demands_v2, M(plk_demands_v2, header) + M(plk_demands_v2, channel_count) + M(plk_demands_v2, channel_capacity) + M(plk_demands_v2, channels) + M(plk_demands_v2, workspace_count) + M(plk_demands_v2, workspace_capacity) + M(plk_demands_v2, workspaces) + M(plk_demands_v2, geometry)),
      L(PLK_ABI_TYPE_ID_plk_tma_tiled_detail_v2, plk_tma_tiled_detail_v2, M(plk_tma_tiled_detail_v2, swizzle) + M(plk_tma_tiled_detail_v2, rank) + M(plk_tma_tiled_detail_v2, box_elements) + M(plk_tma_tiled_detail_v2, element_strides) + M(plk_tma_tiled_detail_v2, reserved)),
      L(PLK_ABI_TYPE_ID_plk_device_resource_v2, plk_device_resource_v2, M(plk_device_resource_v2, channel_id) + M(plk_device_resource_v2, access) + M(plk_device_resource_v2, allocation_address) + M(plk_device_resource_v2, allocation_bytes) + M(plk_device_resource_v2, origin_byte_offset) + M(plk_device_resource_v2, origin_bit_offset) + M(plk_device_resource_v2, domain_id) + M(plk_device_resource_v2, peer_addresses) + M(plk_device_resource_v2, multicast_address)),
      L(PLK_ABI_TYPE_ID_plk_digest_v2, plk_digest_v2, M(plk_digest_v2, sha256)),
      L(PLK_ABI_TYPE_ID_plk_dim3_v2, plk_dim3_v2, M(plk_dim3_v2, x) + M(plk_dim3_v2, y) + M(plk_dim3_v2, z)),
      L(PLK_ABI_TYPE_ID_plk_geometry_v2, plk_geometry_v2, M(plk_geometry_v2, geometry_present) + M(plk_geometry_v2, launch_required) + M(plk_geometry_v2, grid) + M(plk_geometry_v2, block) + M(plk_geometry_v2, cluster) + M(plk_geometry_v2, reserved) + M(plk_geometry_v2, dynamic_smem_bytes)),
      L(PLK_ABI_TYPE_ID_plk_header_v2, plk_header_v2, M(plk_header_v2, abi_version) + M(plk_header_v2, struct_bytes)),
      L(PLK_ABI_TYPE_ID_plk_layout_entry_v2, plk_layout_entry_v2, M(plk_layout_entry_v2, abi_type_id) + M(plk_layout_entry_v2, reserved) + M(plk_layout_entry_v2, bytes) + M(plk_layout_entry_v2, alignment_bytes) + M(plk_layout_entry_v2, compiler_layout)),
      L(PLK_ABI_TYPE_ID_plk_profile_digest_v2, plk_profile_digest_v2, M(plk_profile_digest_v2, dtypes)),
      L(PLK_ABI_TYPE_ID_plk_resources_v2, plk_resources_v2, M(plk_resources_v2, header) + M(plk_resources_v2, channel_count) + M(plk_resources_v2, workspace_count) + M(plk_resources_v2, channels) + M(plk_resources_v2, workspaces) + M(plk_resources_v2, shared) + M(plk_resources_v2, cuda_stream_token) + M(plk_resources_v2, geometry)),
      L(PLK_ABI_TYPE_ID_plk_scalar_v2, plk_scalar_v2, M(plk_scalar_v2, scalar_id) + M(plk_scalar_v2, scalar_type) + M(plk_scalar_v2, value_bits)),
      L(PLK_ABI_TYPE_ID_plk_shared_scalars_v2, plk_shared_scalars_v2, M(plk_shared_scalars_v2, header) + M(plk_shared_scalars_v2, image_bytes) + M(plk_shared_scalars_v2, record_count) + M(plk_shared_scalars_v2, record_offset)),
      L(PLK_ABI_TYPE_ID_plk_transfer_report_v2, plk_transfer_report_v2, M(plk_transfer_report_v2, transfer_id) + M(plk_transfer_report_v2, access) + M(plk_transfer_report_v2, residue_offset) + M(plk_transfer_report_v2, representation_bytes) + M(plk_transfer_report_v2, representation_align) + M(plk_transfer_report_v2, storage_dtype_id) + M(plk_transfer_report_v2, ring_depth) + M(plk_transfer_report_v2, ring_stage_stride_bytes) + M(plk_transfer_report_v2, footprint_bytes_per_stage) + M(plk_transfer_report_v2, credit_bytes_per_stage) + M(plk_transfer_report_v2, source_origin_bits) + M(plk_transfer_report_v2, source_span_bits) + M(plk_transfer_report_v2, vendor_kind) + M(plk_transfer_report_v2, reserved) + M(plk_transfer_report_v2, vendor_detail)),
      L(PLK_ABI_TYPE_ID_plk_tensor_meta_v2, plk_tensor_meta_v2, M(plk_tensor_meta_v2, channel_id) + M(plk_tensor_meta_v2, dtype_id) + M(plk_tensor_meta_v2, rank) + M(plk_tensor_meta_v2, access) + M(plk_tensor_meta_v2, allocation_bytes) + M(plk_tensor_meta_v2, alignment_bytes) + M(plk_tensor_meta_v2, origin_byte_offset) + M(plk_tensor_meta_v2, origin_bit_offset) + M(plk_tensor_meta_v2, reserved) + M(plk_tensor_meta_v2, extents) + M(plk_tensor_meta_v2, bit_strides)),
      L(PLK_ABI_TYPE_ID_plk_workspace_demand_v2, plk_workspace_demand_v2, M(plk_workspace_demand_v2, workspace_id) + M(plk_workspace_demand_v2, reserved) + M(plk_workspace_demand_v2, bytes) + M(plk_workspace_demand_v2, alignment_bytes)),
      L(PLK_ABI_TYPE_ID_plk_workspace_resource_v2, plk_workspace_resource_v2, M(plk_workspace_resource_v2, workspace_id) + M(plk_workspace_resource_v2, reserved) + M(plk_workspace_resource_v2, device_address) + M(plk_workspace_resource_v2, bytes) + M(plk_workspace_resource_v2, alignment_bytes)),
      L(PLK_ABI_TYPE_ID_plk_domain_v2, plk_domain_v2, M(plk_domain_v2, domain_id) + M(plk_domain_v2, rank) + M(plk_domain_v2, world) + M(plk_domain_v2, reserved)),
  };
  const Layout view = L(MOK_ABI_TYPE_ID_MokMxView, MokMxView, M(MokMxView, q) + M(MokMxView, sc) + M(MokMxView, expert_pitch_q) + M(MokMxView, expert_pitch_sc) + M(MokMxView, rows) + M(MokMxView, k) + M(MokMxView, ld_q) + M(MokMxView, ld_sc));
  if (!std::strcmp(owner, "mok_gemm")) {
    v.push_back(L(MOK_ABI_TYPE_ID_MokGemmResidue, MokGemmResidue, M(MokGemmResidue, x) + M(MokGemmResidue, hidden) + M(MokGemmResidue, w_gate) + M(MokGemmResidue, w_up) + M(MokGemmResidue, w_down) + M(MokGemmResidue, row_token) + M(MokGemmResidue, y) + M(MokGemmResidue, ld_y) + M(MokGemmResidue, reserved)));
    v.push_back(view);
  } else if (!std::strcmp(owner, "mok_act")) {
    v.push_back(L(MOK_ABI_TYPE_ID_MokActResidue, MokActResidue, M(MokActResidue, hidden_q) + M(MokActResidue, hidden_sc) + M(MokActResidue, rows) + M(MokActResidue, cols) + M(MokActResidue, ld_q) + M(MokActResidue, ld_sc) + M(MokActResidue, swiglu_limit) + M(MokActResidue, reserved)));
  } else {
    v.push_back(L(MOK_ABI_TYPE_ID_MokFrameworkParams, MokFrameworkParams, M(MokFrameworkParams, tokens_per_expert) + M(MokFrameworkParams, workspace) + M(MokFrameworkParams, num_experts) + M(MokFrameworkParams, op) + M(MokFrameworkParams, num_col_tiles_gate_up) + M(MokFrameworkParams, num_col_tiles_down)));
  }
  return v;
}
#undef M
#undef L

int abi_report(const char* owner, plk_abi_report_v2* out) {
  if (!out || out->header.abi_version != PLK_HOST_ABI_V2 || out->header.struct_bytes != sizeof(*out)) return PLK_E_VERSION;
  const std::vector<Layout> inv = inventory(owner);
  if (out->entry_capacity != inv.size() || !out->entries) return PLK_E_CAPACITY;
  for (size_t i = 0; i < inv.size(); ++i)
    if (out->entries[i].abi_type_id != inv[i].id) return PLK_E_CONTRACT;
  for (size_t i = 0; i < inv.size(); ++i) {
    out->entries[i].reserved = 0;
    out->entries[i].bytes = inv[i].bytes;
    out->entries[i].alignment_bytes = inv[i].align;
    out->entries[i].compiler_layout = Sha256::of(inv[i].text);
  }
  out->entry_count = (uint32_t)inv.size();
  out->profile.dtypes = Sha256::of("u8:8;i32:32;bf16:16;e4m3:8;e8m0:8;");
  out->owner_contract = Sha256::of(std::string("pipelink-amd/") + owner + "/mxfp8-fwd/1");
  return PLK_OK;
}

// ---- shared scalars -> dimensions -------------------------------------------------------------
bool read_dims(const plk_shared_scalars_v2* shared, plk_mok::Dims& d) {
  if (!shared || shared->header.abi_version != PLK_HOST_ABI_V2 || shared->header.struct_bytes != sizeof(*shared)) return false;
  if ((uint64_t)shared->record_offset + (uint64_t)shared->record_count * sizeof(plk_scalar_v2) > shared->image_bytes) return false;
  const auto* rec = reinterpret_cast<const plk_scalar_v2*>(reinterpret_cast<const unsigned char*>(shared) + shared->record_offset);
  int64_t v[66] = {};
  uint64_t seen = 0;
  double limit = 0;
  bool have_limit = false;
  for (uint32_t i = 0; i < shared->record_count; ++i) {
    const uint32_t id = rec[i].scalar_id;
    if (id == MOK_SCALAR_SWIGLU_LIMIT) {
      if (rec[i].scalar_type != PLK_SCALAR_F64) return false;
      std::memcpy(&limit, &rec[i].value_bits, 8);
      have_limit = true;
      continue;
    }
    const bool known = (id >= 1 && id <= 4) || id == MOK_SCALAR_PASS || id == MOK_SCALAR_PRECISION || (id >= 60 && id <= 65);
    if (!known) continue;  // other owners' scalars
    if (rec[i].scalar_type != PLK_SCALAR_I64) return false;
    std::memcpy(&v[id], &rec[i].value_bits, 8);
    if (v[id] < 0 || v[id] > INT32_MAX) return false;
    seen |= 1ull << (id >= 60 ? id - 40 : id);  // ids 60..65 -> bits 20..25
  }
  for (uint32_t id : {1u, 2u, 3u, 4u, 11u, 12u, 60u, 61u, 62u, 63u, 64u, 65u})
    if (!(seen & (1ull << (id >= 60 ? id - 40 : id)))) return false;
  if (!have_limit || v[MOK_SCALAR_PRECISION] != 1 || v[MOK_SCALAR_PASS] < 0 || v[MOK_SCALAR_PASS] > 2) return false;
  d.tokens = (int32_t)v[MOK_SCALAR_NUM_LOCAL_TOKENS];
  d.hidden = (int32_t)v[MOK_SCALAR_HIDDEN];
  d.intermediate = (int32_t)v[MOK_SCALAR_INTERMEDIATE];
  d.experts = (int32_t)v[MOK_SCALAR_NUM_LOCAL_EXPERTS];
  d.routed_rows = (int32_t)v[MOK_SCALAR_ROUTED_ROWS];
  d.ld_q_h = (int32_t)v[MOK_SCALAR_LD_Q_H];
  d.ld_q_i = (int32_t)v[MOK_SCALAR_LD_Q_I];
  d.ld_sc_h = (int32_t)v[MOK_SCALAR_LD_SC_H];
  d.ld_sc_i = (int32_t)v[MOK_SCALAR_LD_SC_I];
  d.pass = (int32_t)v[MOK_SCALAR_PASS];
  d.swiglu_limit = (float)limit;
  if (v[MOK_SCALAR_WORKSPACE_WORDS] != plk_mok::workspace_words(d)) return false;
  if (d.pass == 0 && d.ld_q_i % 128) return false;  // one launch for both GEMMs wants whole cache lines per row of `hidden`
  return plk_mok::check_dims(d) == nullptr;
}

struct Shape {
  uint32_t rank, bits, access;
  uint64_t extents[4];
};

Shape channel_shape(const char* owner, uint32_t id, const plk_mok::Dims& d) {
  const uint64_t T = d.tokens, H = d.hidden, I = d.intermediate, E = d.experts, R = d.routed_rows;
  if (!std::strcmp(owner, "mok_gemm")) {
    switch (id) {
      case 1: return {2, 8, PLK_ACCESS_READ, {T, (uint64_t)d.ld_q_h}};
      case 2: return {2, 8, PLK_ACCESS_READ, {T, (uint64_t)d.ld_sc_h}};
      case 3: case 5: return {4, 8, PLK_ACCESS_READ, {E, H / 64, I, 64}};
      case 4: case 6: return {4, 8, PLK_ACCESS_READ, {E, (H + 127) / 128, I, 4}};
      case 7: return {4, 8, PLK_ACCESS_READ, {E, I / 64, H, 64}};
      case 8: return {4, 8, PLK_ACCESS_READ, {E, (I + 127) / 128, H, 4}};
      case 9: return {2, 8, PLK_ACCESS_READ, {R, (uint64_t)d.ld_q_i}};
      case 10: return {2, 8, PLK_ACCESS_READ, {R, (uint64_t)d.ld_sc_i}};
      case 11: return {2, 16, PLK_ACCESS_WRITE, {R, H}};
      case 12: return {1, 32, PLK_ACCESS_READ, {R}};
    }
  } else if (!std::strcmp(owner, "mok_act")) {
    switch (id) {
      case 1: return {2, 8, PLK_ACCESS_WRITE, {R, (uint64_t)d.ld_q_i}};
      case 2: return {2, 8, PLK_ACCESS_WRITE, {R, (uint64_t)d.ld_sc_i}};
    }
  } else if (id == 1) {
    return {1, 32, PLK_ACCESS_READ, {E}};
  } else if (id == 2) {
    return {1, 32, PLK_ACCESS_WRITE, {(uint64_t)plk_mok::workspace_words(d)}};
  }
  return {};
}
uint32_t channel_count_of(const char* owner) {
  return !std::strcmp(owner, "mok_gemm") ? MOK_GEMM_CHANNEL_COUNT : !std::strcmp(owner, "mok_act") ? MOK_ACT_CHANNEL_COUNT : MOK_FRAMEWORK_CHANNEL_COUNT;
}
uint64_t byte_size(const Shape& s) {
  uint64_t b = s.bits / 8;
  for (uint32_t i = 0; i < s.rank; ++i) b *= s.extents[i];
  return b;
}
bool optional_channel(const char* owner, uint32_t id) { return !std::strcmp(owner, "mok_gemm") && id == 12; }

bool topology_ok(const plk_common_v2& c) {
  return c.block.x == plk_mok::THREADS && c.block.y == 1 && c.block.z == 1 && c.cluster.x == 1 && c.cluster.y == 1 && c.cluster.z == 1;
}

int query(const char* owner, const plk_common_v2* common, const void* args, plk_demands_v2* out) {
  if (!common || args || !out) return PLK_E_ARGUMENT;
  if (common->header.abi_version != PLK_HOST_ABI_V2 || common->header.struct_bytes != sizeof(*common) ||
      out->header.abi_version != PLK_HOST_ABI_V2 || out->header.struct_bytes != sizeof(*out))
    return PLK_E_VERSION;
  if (!topology_ok(*common)) return PLK_E_CONTRACT;
  const uint32_t n = channel_count_of(owner);
  if (common->channel_count != n || !common->channels || out->channel_capacity != n || !out->channels || out->workspace_capacity)
    return PLK_E_CONTRACT;
  plk_mok::Dims d;
  if (!read_dims(common->shared, d)) return PLK_E_ARGUMENT;
  for (uint32_t i = 0; i < n; ++i) {
    const plk_tensor_meta_v2& src = common->channels[i];
    plk_channel_demand_v2& dem = out->channels[i];
    Shape s = channel_shape(owner, i + 1, d);
    if (src.channel_id != i + 1 || dem.channel_id != i + 1 || src.rank != s.rank || dem.rank != s.rank || src.access != s.access ||
        !src.extents || !src.bit_strides || !dem.extents || !dem.bit_strides)
      return PLK_E_CONTRACT;
    // an optional channel may be declared empty (all extents zero)
    if (optional_channel(owner, i + 1) && src.extents[0] == 0) s.extents[0] = 0;
    const uint64_t bytes = byte_size(s);
    dem.dtype_id = src.dtype_id;
    dem.access = s.access;
    dem.minimum_allocation_bytes = bytes;
    dem.alignment_bytes = s.bits == 32 ? 4 : 16;
    int64_t stride = bytes ? (int64_t)s.bits : 0;
    for (int k = (int)s.rank - 1; k >= 0; --k) {
      if (src.extents[k] != s.extents[k] || src.bit_strides[k] != stride) return PLK_E_ARGUMENT;  // dense, in the demanded shape
      dem.extents[k] = s.extents[k];
      dem.bit_strides[k] = stride;
      stride *= (int64_t)s.extents[k];
    }
  }
  out->channel_count = n;
  out->workspace_count = 0;
  out->geometry = plk_geometry_v2{};
  if (!std::strcmp(owner, "mok_framework")) {  // the schedule's owner states the launch: one workgroup per CU is the caller's to cap
    out->geometry.geometry_present = 1;
    out->geometry.launch_required = 1;
    out->geometry.grid = {(uint32_t)plk_mok::max_workgroups(d), 1, 1};
    out->geometry.block = {plk_mok::THREADS, 1, 1};
    out->geometry.cluster = {1, 1, 1};
    out->geometry.dynamic_smem_bytes = common->dynamic_smem_bytes;
  }
  return PLK_OK;
}

int build(const char* owner, const plk_common_v2* common, const void* args, const plk_resources_v2* res, void* residue,
          size_t cap, uint32_t transfer_capacity, plk_session** session) {
  if (!session) return PLK_E_ARGUMENT;
  *session = nullptr;
  if (!common || args || !res || !residue) return PLK_E_ARGUMENT;
  if (common->header.abi_version != PLK_HOST_ABI_V2 || common->header.struct_bytes != sizeof(*common) ||
      res->header.abi_version != PLK_HOST_ABI_V2 || res->header.struct_bytes != sizeof(*res))
    return PLK_E_VERSION;
  const bool gemm = !std::strcmp(owner, "mok_gemm"), act = !std::strcmp(owner, "mok_act");
  const size_t need = gemm ? sizeof(MokGemmResidue) : act ? sizeof(MokActResidue) : sizeof(MokFrameworkParams);
  if (cap < need || transfer_capacity) return PLK_E_CAPACITY;
  const uint32_t n = channel_count_of(owner);
  if (res->channel_count != n || !res->channels || res->workspace_count) return PLK_E_CONTRACT;
  plk_mok::Dims d;
  if (!read_dims(res->shared, d)) return PLK_E_ARGUMENT;
  uint64_t addr[MOK_GEMM_CHANNEL_COUNT] = {};
  for (uint32_t i = 0; i < n; ++i) {
    const plk_device_resource_v2& r = res->channels[i];
    const Shape s = channel_shape(owner, i + 1, d);
    const uint64_t bytes = byte_size(s);
    if (r.channel_id != i + 1 || r.origin_bit_offset || r.origin_byte_offset > r.allocation_bytes) return PLK_E_RESOURCE;
    if (optional_channel(owner, i + 1) && !r.allocation_address && !r.allocation_bytes) continue;  // absent: rows are tokens
    if (bytes > r.allocation_bytes - r.origin_byte_offset) return PLK_E_RESOURCE;
    if (!bytes) continue;
    if (!r.allocation_address || r.allocation_address > UINT64_MAX - r.origin_byte_offset) return PLK_E_RESOURCE;
    addr[i] = r.allocation_address + r.origin_byte_offset;
    if (addr[i] % (s.bits == 32 ? 4 : 16)) return PLK_E_RESOURCE;
  }
  std::memset(residue, 0, need);
  if (gemm) {
    if (d.pass == 0 && !plk_mok::one_launch_ok(d, addr[8])) return PLK_E_RESOURCE;  // hidden_q rows must be whole cache lines
    plk_mok::GemmAddresses a{addr[0], addr[1], addr[2], addr[3], addr[4], addr[5], addr[6], addr[7], addr[8], addr[9], addr[10], addr[11]};
    const MokGemmResidue g = plk_mok::gemm_residue(d, a);
    std::memcpy(residue, &g, sizeof g);
  } else if (act) {
    const MokActResidue a = plk_mok::act_residue(d, addr[0], addr[1]);
    std::memcpy(residue, &a, sizeof a);
  } else {
    const MokFrameworkParams f = plk_mok::framework_params(d, addr[0], addr[1]);
    std::memcpy(residue, &f, sizeof f);
  }
  return PLK_OK;
}

}  // namespace

#define PLK_DEFINE_OWNER(suffix)                                                                                              \
  extern "C" int pipelink_params_abi_##suffix(plk_abi_report_v2* out) { return abi_report(#suffix, out); }                    \
  extern "C" int pipelink_params_query_##suffix(const plk_common_v2* c, const void* a, plk_demands_v2* o) {                   \
    return query(#suffix, c, a, o);                                                                                           \
  }                                                                                                                           \
  extern "C" int pipelink_params_build_##suffix(const plk_common_v2* c, const void* a, const plk_resources_v2* r, void* out,  \
                                                size_t cap, plk_transfer_report_v2*, uint32_t tcap, plk_session** s) {        \
    return build(#suffix, c, a, r, out, cap, tcap, s);                                                                        \
  }                                                                                                                           \
  extern "C" int pipelink_params_release_##suffix(plk_session* s) { return s ? PLK_E_RELEASE : PLK_OK; }
PLK_DEFINE_OWNER(mok_gemm)
PLK_DEFINE_OWNER(mok_act)
PLK_DEFINE_OWNER(mok_framework)
