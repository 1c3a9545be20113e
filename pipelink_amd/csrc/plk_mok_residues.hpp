// What the routed-expert FFN pipeline's three owners read at run time, built from problem
// dimensions and device addresses.  One place for the forward entry (plk_mok.cpp) and the
// host-ABI providers (plk_mok_provider.cpp), so both hand the kernel the same bytes.
#ifndef PLK_MOK_RESIDUES_HPP
#define PLK_MOK_RESIDUES_HPP

#include <cstdint>
#include <vector>

#include "../stages/mok/include/mok_abi.h"

namespace plk_mok {

constexpr int TILE_X = 256;  // routed rows per workgroup tile   (fact mok.gemm.TILE_X)
constexpr int TILE_W = 256;  // weight rows per workgroup tile   (fact mok.gemm.TILE_W)
constexpr int K_STEP = 64;   // contraction bytes per MFMA step  (fact mok.gemm.K_SLOT)
constexpr int MAX_EXPERTS = 256;
constexpr int NUM_XCD = 8;
constexpr uint32_t THREADS = 256;

struct Dims {
  int32_t tokens = 0, hidden = 0, intermediate = 0, experts = 0, routed_rows = 0;
  int32_t ld_q_h = 0, ld_q_i = 0;    // code row pitch of x / hidden, bytes
  int32_t ld_sc_h = 0, ld_sc_i = 0;  // scale row pitch of x / hidden
  int32_t pass = 0;                  // 0 = both GEMMs in one launch, 1 = gate/up + SwiGLU + requant, 2 = down
  float swiglu_limit = 7.0f;
};

// nullptr if the dimensions are ones the kernel handles, else what is wrong with them
inline const char* check_dims(const Dims& d) {
  if (d.experts <= 0 || d.experts > MAX_EXPERTS) return "num_experts must be in 1..256";
  if (d.hidden <= 0 || d.intermediate <= 0 || d.hidden % K_STEP || d.intermediate % K_STEP)
    return "hidden and intermediate must be positive multiples of 64";
  if (d.ld_sc_h % 16 || d.ld_sc_i % 16 || d.ld_sc_h * 32 < d.hidden || d.ld_sc_i * 32 < d.intermediate)
    return "scale pitch must be a multiple of 16 covering K/32 blocks";
  if (d.ld_q_h < d.hidden || d.ld_q_h % 16 || d.ld_q_i < d.intermediate || d.ld_q_i % 16)
    return "code row pitch must be a multiple of 16 and at least K";
  if (d.tokens < 0 || d.routed_rows < 0) return "negative row count";
  // the kernel addresses one operand with 32-bit byte offsets from its base
  // and marks rows past the end of a tile with an offset in the last 16 MiB of that range
  const int64_t lim = ((int64_t)1 << 32) - ((int64_t)1 << 24);
  if ((int64_t)d.tokens * d.ld_q_h >= lim || (int64_t)d.routed_rows * d.ld_q_i >= lim || (int64_t)d.intermediate * d.hidden >= lim)
    return "an operand (rows x row pitch) must stay 16 MiB below 4 GiB";
  return nullptr;
}

// activations: row-major codes with pitch ld_q, row-major scales with pitch ld_sc;
// weights (per_expert): K-tiled codes [K/64, rows, 64], slot-major scales [K/128, rows, 4]
inline MokMxView mx_view(uint64_t q, uint64_t sc, int64_t rows, int k, int ld_q, int ld_sc, bool per_expert) {
  MokMxView v{};
  v.q = (const uint8_t*)(uintptr_t)q;
  v.sc = (const uint8_t*)(uintptr_t)sc;
  v.rows = (int32_t)rows;
  v.k = k;
  v.ld_q = per_expert ? 64 : ld_q;
  v.ld_sc = ld_sc;
  v.expert_pitch_q = per_expert ? rows * (int64_t)k : 0;
  v.expert_pitch_sc = per_expert ? (int64_t)((k + 127) / 128) * rows * 4 : 0;
  return v;
}

struct GemmAddresses {
  uint64_t x_q, x_sc, w_gate_q, w_gate_sc, w_up_q, w_up_sc, w_down_q, w_down_sc, hidden_q, hidden_sc, y, row_token;
};

inline MokGemmResidue gemm_residue(const Dims& d, const GemmAddresses& a) {
  MokGemmResidue g{};
  const int H = d.hidden, I = d.intermediate;
  g.x = mx_view(a.x_q, a.x_sc, d.tokens, H, d.ld_q_h, d.ld_sc_h, false);
  g.hidden = mx_view(a.hidden_q, a.hidden_sc, d.routed_rows, I, d.ld_q_i, d.ld_sc_i, false);
  g.w_gate = mx_view(a.w_gate_q, a.w_gate_sc, I, H, 0, d.ld_sc_h, true);
  g.w_up = mx_view(a.w_up_q, a.w_up_sc, I, H, 0, d.ld_sc_h, true);
  g.w_down = mx_view(a.w_down_q, a.w_down_sc, H, I, 0, d.ld_sc_i, true);
  g.row_token = (const int32_t*)(uintptr_t)a.row_token;
  g.y = (uint16_t*)(uintptr_t)a.y;
  g.ld_y = H;
  return g;
}

inline MokActResidue act_residue(const Dims& d, uint64_t hidden_q, uint64_t hidden_sc) {
  MokActResidue a{};
  a.hidden_q = (uint8_t*)(uintptr_t)hidden_q;
  a.hidden_sc = (uint8_t*)(uintptr_t)hidden_sc;
  a.rows = d.routed_rows;
  a.cols = d.intermediate;
  a.ld_q = d.ld_q_i;
  a.ld_sc = d.ld_sc_i;
  a.swiglu_limit = d.swiglu_limit;
  return a;
}

inline int32_t num_col_tiles_gate_up(const Dims& d) { return (d.intermediate + TILE_W / 2 - 1) / (TILE_W / 2); }
inline int32_t num_col_tiles_down(const Dims& d) { return (d.hidden + TILE_W - 1) / TILE_W; }

// an upper bound of the number of routed-row tiles: every expert may end in a partial tile
inline int64_t max_row_tiles(const Dims& d) { return ((int64_t)d.routed_rows + TILE_X - 1) / TILE_X + d.experts; }

// 32-bit words of the launch workspace (MOK_WS_* words, then one readiness counter per routed-row tile)
inline int64_t workspace_words(const Dims& d) { return MOK_WS_COUNTERS + max_row_tiles(d); }

// One launch may run both GEMMs only if no cache line of `hidden` is shared between two gate/up tiles, whose
// workgroups may sit on different XCDs: rows that start and end on 128-byte boundaries (a gate/up tile writes 128
// bytes of a row).  Otherwise the forward is two launches.
inline bool one_launch_ok(const Dims& d, uint64_t hidden_q) { return d.ld_q_i % 128 == 0 && hidden_q % 128 == 0; }

inline MokFrameworkParams framework_params(const Dims& d, uint64_t tokens_per_expert, uint64_t workspace) {
  MokFrameworkParams fw{};
  fw.tokens_per_expert = (const int32_t*)(uintptr_t)tokens_per_expert;
  fw.workspace = (uint32_t*)(uintptr_t)workspace;
  fw.num_experts = d.experts;
  fw.op = d.pass == 0 ? MOK_FWD_BOTH : d.pass == 1 ? MOK_GEMM_FWD_ROUTED_GATE_UP : MOK_GEMM_FWD_ROUTED_DOWN;
  fw.num_col_tiles_gate_up = num_col_tiles_gate_up(d);
  fw.num_col_tiles_down = num_col_tiles_down(d);
  return fw;
}

// an upper bound of the number of tiles of the launch: more workgroups than this would idle
inline int64_t max_workgroups(const Dims& d) {
  return max_row_tiles(d) * ((d.pass != 2 ? num_col_tiles_gate_up(d) : 0) + (d.pass != 1 ? num_col_tiles_down(d) : 0));
}

}  // namespace plk_mok

#endif
