// Stage package mok.framework: the persistent worker role.  It owns the schedule (which
// workgroup runs which tile, in which order) and calls the GEMM and activation owners
// through link-generated trampolines; it knows nothing of their tile internals beyond the
// published facts TILE_X / TILE_W.
//
// Plays the part of mok_framework_run in campaigns/mok/port/framework/interp_fwd.cu:26-252
// (task decode :137-214).  Not carried over: CLC work stealing and 2-CTA clusters (no
// gfx950 counterpart) and the comm clusters (single GPU).  The schedule here is static:
// tiles are numbered expert-major, within one expert column-tile-major with the row tiles
// innermost, so workgroups that run at the same time share one weight tile; the tile
// range is split in 8 contiguous chunks, one per XCD (workgroup id % 8), so each L2 sees
// a contiguous run of experts.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "../include/mok_device.hpp"

extern "C" __device__ int pipelink_mok_fw_sched();  // byte offset of the schedule table in dynamic LDS

extern "C" __device__ void pipelink_call_gemm_init(const void* view);
extern "C" __device__ void pipelink_call_act_init(const void* view);
extern "C" __device__ void pipelink_call_gemm_prefetch(const void* view, const MokGemmTask*, mok::GemmCarry*);
extern "C" __device__ void pipelink_call_gemm_fwd(const void* view, const MokGemmTask*, const MokCounters*, uint32_t*,
                                                  mok::AccFrag*, const mok::GemmCarry*);
extern "C" __device__ void pipelink_call_gemm_store(const void* view, const MokGemmTask*, const mok::AccFrag*);
extern "C" __device__ void pipelink_call_act_fwd(const void* view, const MokActTask*, const MokCounters*, uint32_t*,
                                                 const mok::AccFrag*);

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mok_framework {
constexpr int MAX_EXPERTS = 256;
constexpr int NUM_XCD = 8;
}

extern "C" __device__ void mok_framework_worker(const void* params, unsigned variant) {
  (void)variant;
  using namespace mok_framework;
  const pipelink_host_view view{params, nullptr};
  const MokFrameworkParams& g = *static_cast<const MokFrameworkParams*>(params);
  int* row_begin = reinterpret_cast<int*>(pipelink_smem + pipelink_mok_fw_sched());
  int* tile_begin = row_begin + (MAX_EXPERTS + 1);
  const int ne = g.num_experts;

  pipelink_call_gemm_init(&view);
  pipelink_call_act_init(&view);

  // exclusive prefix sums of rows and row tiles per expert (every workgroup computes its own copy)
  if (threadIdx.x == 0) {
    int rows = 0, tiles = 0;
    for (int e = 0; e < ne; ++e) {
      row_begin[e] = rows;
      tile_begin[e] = tiles;
      const int c = g.tokens_per_expert[e];
      rows += c;
      tiles += (c + mok::TILE_X - 1) / mok::TILE_X;
    }
    row_begin[ne] = rows;
    tile_begin[ne] = tiles;
  }
  __syncthreads();

  const int nct = g.num_col_tiles;
  const int total = tile_begin[ne] * nct;
  const int chunk = (total + NUM_XCD - 1) / NUM_XCD;
  const int xcd = blockIdx.x % NUM_XCD;
  const int per_xcd = gridDim.x / NUM_XCD;  // launch grid is a multiple of NUM_XCD
  const int chunk_end = min(total, (xcd + 1) * chunk);
  const MokCounters counters{nullptr};
  uint32_t phase = 0;

  const bool gate_up = g.op == MOK_GEMM_FWD_ROUTED_GATE_UP;
  auto decode = [&](int idx) {
    // expert of tile idx: last e with tile_begin[e] * nct <= idx
    int lo = 0, hi = ne;
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (tile_begin[mid] * nct <= idx) lo = mid; else hi = mid;
    }
    const int e = __builtin_amdgcn_readfirstlane(lo);
    const int mtiles = tile_begin[e + 1] - tile_begin[e];
    const int local = idx - tile_begin[e] * nct;
    const int nt = local / mtiles;
    const int mt = local - nt * mtiles;
    const int col_begin = nt * (gate_up ? mok::TILE_W / 2 : mok::TILE_W);
    // wave-uniform by construction; say so, so that the task lives in scalar registers
    return MokGemmTask{g.op, e, __builtin_amdgcn_readfirstlane(row_begin[e] + mt * mok::TILE_X),
                       __builtin_amdgcn_readfirstlane(row_begin[e + 1]), __builtin_amdgcn_readfirstlane(col_begin), idx, 0u};
  };

  // Software pipeline over this workgroup's tiles: the next tile's first loads are issued
  // between a tile's mainloop and its epilogue, so they fly while the epilogue computes.
  int idx = xcd * chunk + blockIdx.x / NUM_XCD;
  if (idx >= chunk_end) return;
  MokGemmTask task = decode(idx);
  mok::GemmCarry carry;
  pipelink_call_gemm_prefetch(&view, &task, &carry);
  for (;;) {
    const int next_idx = idx + per_xcd;
    const bool has_next = next_idx < chunk_end;
    MokGemmTask next = task;
    if (has_next) next = decode(next_idx);
    mok::AccFrag acc;
    pipelink_call_gemm_fwd(&view, &task, &counters, &phase, &acc, &carry);
    if (has_next) pipelink_call_gemm_prefetch(&view, &next, &carry);
    if (gate_up) {
      const MokActTask act{MOK_ACT_FWD_ROUTED, task.row_begin, task.row_end, task.col_begin, idx, 0u};
      pipelink_call_act_fwd(&view, &act, &counters, &phase, &acc);
    } else {
      pipelink_call_gemm_store(&view, &task, &acc);
    }
    if (!has_next) break;
    task = next;
    idx = next_idx;
  }
}
#else  // PIPELINK_EMIT: host-evaluated annotations only
#include "../include/mok_abi.h"
#endif

PL_STAGE("mok.framework", "0.1.0");
PL_PARAMS(MokFrameworkParams);
PL_ROLE(worker, mok_framework_worker, 4);
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_CALL(gemm_init, "mok_gemm_init", "extern \"C\" __device__ void pipelink_call_gemm_init(const void* view);");
PL_CALL(act_init, "mok_act_init", "extern \"C\" __device__ void pipelink_call_act_init(const void* view);");
PL_CALL(gemm_prefetch, "mok_gemm_prefetch",
        "extern \"C\" __device__ void pipelink_call_gemm_prefetch(const void* view, const MokGemmTask* task, mok::GemmCarry* carry);");
PL_CALL(gemm_fwd, "mok_gemm_fwd",
        "extern \"C\" __device__ void pipelink_call_gemm_fwd(const void* view, const MokGemmTask* task, "
        "const MokCounters* counters, uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry);");
PL_CALL(gemm_store, "mok_gemm_store",
        "extern \"C\" __device__ void pipelink_call_gemm_store(const void* view, const MokGemmTask* task, const mok::AccFrag* acc);");
PL_CALL(act_fwd, "mok_act_fwd",
        "extern \"C\" __device__ void pipelink_call_act_fwd(const void* view, const MokActTask* task, "
        "const MokCounters* counters, uint32_t* phase, const mok::AccFrag* acc);");
// schedule table: exclusive prefix sums of rows and row tiles for up to 256 experts
PL_CLAIM("pipelink_mok_fw_sched", "smem", 2 * (256 + 1) * 4, 16, "kernel");
PL_USES("pipelink_mok_fw_sched");
// host contract: the schedule's owner
PL_HOST_GROUP("mok.framework.params", "mok_framework");
PL_HOST_ABI_TYPE(3, MokFrameworkParams);
MOK_HOST_SCALARS();
PL_HOST_CHANNEL(1, "tokens_per_expert", 32, "read", "mok.num_local_experts", false);
PL_FACT("mok.framework.MAX_EXPERTS", 256);
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
