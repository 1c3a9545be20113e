// Package oe.loader.wide: fills the LDS ring of the wide matrix package (256 A rows + 128 B^T rows per stage).
//
// Three waves: waves 0 and 1 bring the upper and lower 128 of the tile's A rows, wave 2 its 128 B^T rows.  A ring
// stage holds 64 contraction elements (128 bytes) of the 256 A rows, then of the 128 B^T rows: 48 KB, so a ring of
// three stages is what 160 KB of LDS hold.  Loads, swizzle and hand-shake are those of the three-package example's
// loader (one buffer_load_dwordx4 ... lds moves 8 rows; lane i lands at byte 16 * i of the 1 KB piece and fetches the
// chunk that belongs there under  position = chunk ^ (row % 8)); a wave has 16 loads per stage and runs one stage
// ahead of the stage it reports full.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <pipelink/ring.hpp>
#include "include/oe_abi.h"

extern "C" __device__ int pipelink_gs_depth();      // ring stages, bound at link time
extern "C" __device__ int pipelink_gs_ring();       // byte offset of the ring in dynamic LDS
extern "C" __device__ int pipelink_gs_full();       // first 16-byte slot of the full counters
extern "C" __device__ int pipelink_gs_empty();      // first 16-byte slot of the empty counters
extern "C" __device__ int pipelink_oe_warp_load();  // index of this role's first wave in the workgroup

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace oe_loader_wide {
typedef __attribute__((address_space(3))) void* lds_ptr;
constexpr int ROWS_PER_WAVE = 128;
constexpr int LOADS_PER_STAGE = ROWS_PER_WAVE / 8;  // 16 per wave
constexpr int MMA_WAVES = 4;

template <int AHEAD>
__device__ __forceinline__ void wait_stages() { pl::ring_wait_loads<AHEAD * LOADS_PER_STAGE>(); }
__device__ __forceinline__ void wait_stages(int stages_in_flight) {
  switch (stages_in_flight) {
    case 3: wait_stages<3>(); break;
    case 2: wait_stages<2>(); break;
    case 1: wait_stages<1>(); break;
    default: wait_stages<0>(); break;
  }
}
}  // namespace oe_loader_wide

extern "C" __device__ void oe_loader_wide_role_load(const void* params, unsigned variant) {
  (void)variant;
  using namespace oe_loader_wide;
  const OeLoaderParams& p = *static_cast<const OeLoaderParams*>(params);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) - pipelink_oe_warp_load();
  const int operand = wave >> 1;  // 0: A rows (wave = upper or lower 128 of them), 1: B^T rows
  const int depth = pipelink_gs_depth();
  unsigned char* ring = pipelink_smem + pipelink_gs_ring() + wave * (ROWS_PER_WAVE * 128);
  const int tiles_n = p.n / OE_WIDE_TILE_N;
  const int row0 = operand == 0 ? (int)(blockIdx.x / tiles_n) * OE_WIDE_TILE_M + wave * ROWS_PER_WAVE : (int)(blockIdx.x % tiles_n) * OE_WIDE_TILE_N;
  const uint32_t row_pitch = (uint32_t)p.k * 2u;
  const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(operand == 0 ? p.a : p.bt), 0,
                                                                        (int)((uint32_t)(operand == 0 ? p.m : p.n) * row_pitch), 0x00020000);
  const int r8 = lane >> 3, pos = lane & 7;
  // rows of one load are 8 consecutive rows starting at a multiple of 8
  const uint32_t lane_offset = (uint32_t)(row0 + r8) * row_pitch + 16u * (uint32_t)(pos ^ r8);
  const int stages = p.k / OE_TILE_K;
  // stages in flight behind the one being issued: a stage may only be refilled once it is read, so depth - 1 at
  // most, and one less leaves a free stage between this role and the readers (with none, every fill waits for a
  // hand-shake: 1.98 ms against 1.18 ms for the 8192^3 product)
  const int ahead = depth <= 2 ? 1 : (depth - 2 < 3 ? depth - 2 : 3);
  bool ok = true;
  for (int s = 0; s < stages; ++s) {
    const int slot = s % depth, fill = s / depth;
    // the stage's previous contents have been read by every mma wave
    if (fill > 0) ok &= pl::ring_wait(pl::ring_counter(pipelink_smem, pipelink_gs_empty(), slot), (uint32_t)fill * MMA_WAVES);
    unsigned char* stage = ring + slot * OE_WIDE_STAGE_BYTES;
#pragma unroll
    for (int i = 0; i < LOADS_PER_STAGE; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, (lds_ptr)(stage + i * 1024), 16, (int)(lane_offset + i * 8 * row_pitch),
                                               (int)((uint32_t)s * 128u), 0, 0);
    if (s >= ahead) {
      wait_stages(ahead);  // everything but the youngest `ahead` stages has landed
      if (lane == 0) pl::ring_arrive(pl::ring_counter(pipelink_smem, pipelink_gs_full(), (s - ahead) % depth));
    }
  }
  for (int t = stages > ahead ? stages - ahead : 0; t < stages; ++t) {  // the last stages, oldest first
    wait_stages(stages - 1 - t);
    if (lane == 0) pl::ring_arrive(pl::ring_counter(pipelink_smem, pipelink_gs_full(), t % depth));
  }
  if (!ok && lane == 0) atomicOr(p.status, 1u);
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.loader.wide", "0.1.0");
PL_PARAMS(OeLoaderParams);
PL_ROLE(load, oe_loader_wide_role_load, OE_WIDE_LOAD_WAVES);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
// ring stage = 384 rows (256 of A, 128 of B^T) x 64 bf16
PL_RING(ab_ring, "produce", load, "bf16", 16, 384, 64, "pipelink_gs_depth", OE_WIDE_STAGE_BYTES, "pipelink_gs_full", "warps(load)", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_RING("pipelink_gs_ring", "smem", 0, "pipelink_gs_depth", OE_WIDE_STAGE_BYTES, 1024, "kernel");
PL_CLAIM_RING("pipelink_gs_full", "mbarrier", 0, "pipelink_gs_depth", 1, 1, "kernel");
PL_CLAIM_RING("pipelink_gs_empty", "mbarrier", 0, "pipelink_gs_depth", 1, 1, "kernel");
PL_CLAIM_WARPS("pipelink_oe_warp_load", load, OE_WIDE_LOAD_WAVES);
PL_USES("pipelink_oe_warp_load");
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
