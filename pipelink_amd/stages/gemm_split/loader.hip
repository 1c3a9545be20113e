// Package gs.loader: fills the LDS ring of the three-package GEMM example.
//
// Two waves: wave 0 brings the tile's 128 A rows, wave 1 its 128 B^T rows.  A ring stage holds 64
// contraction elements (128 bytes) of the A rows, then of the B^T rows.  One buffer_load_dwordx4 ... lds
// moves 8 rows: lane i lands at byte 16 * i of the 1 KB piece, i.e. row i / 8, 16-byte position i % 8, and
// fetches the chunk that belongs there under the swizzle  position = chunk ^ (row % 8)  the mma role reads
// with.  A wave has 16 loads per stage and runs up to 3 stages ahead (fewer in a short ring): it issues stage s, then
// waits until all but the youngest 16 * ahead loads have landed (s_waitcnt vmcnt: a wave cannot have more
// than 63 loads in flight, which is why there are two waves) and arrives on the `full` counter of stage
// s - ahead.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <pipelink/ring.hpp>
#include "include/gs_abi.h"

extern "C" __device__ int pipelink_gs_depth();  // ring stages, bound at link time
extern "C" __device__ int pipelink_gs_ring();   // byte offset of the ring in dynamic LDS
extern "C" __device__ int pipelink_gs_full();   // first 16-byte slot of the full counters
extern "C" __device__ int pipelink_gs_empty();  // first 16-byte slot of the empty counters
extern "C" __device__ int pipelink_gs_warp_load();  // index of this role's first wave in the workgroup

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace gs_loader {
typedef __attribute__((address_space(3))) void* lds_ptr;
constexpr int LOADS_PER_STAGE = GS_TILE_M / 8;  // 16 per wave

// this wave's half of a stage: `rows` is A (wave 0) or B^T (wave 1), `half_stage` where its rows go
__device__ __forceinline__ void issue_stage(__amdgpu_buffer_rsrc_t rows, uint32_t lane_offset, uint32_t row_pitch, uint32_t kbyte,
                                            unsigned char* half_stage) {
#pragma unroll
  for (int i = 0; i < LOADS_PER_STAGE; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rows, (lds_ptr)(half_stage + i * 1024), 16, (int)(lane_offset + i * 8 * row_pitch), (int)kbyte, 0, 0);
}
// at most `stages_in_flight` of this wave's stages still on their way (s_waitcnt takes an immediate)
__device__ __forceinline__ void wait_stages(int stages_in_flight) {
  switch (stages_in_flight) {
    case 3: pl::ring_wait_loads<3 * LOADS_PER_STAGE>(); break;
    case 2: pl::ring_wait_loads<2 * LOADS_PER_STAGE>(); break;
    case 1: pl::ring_wait_loads<LOADS_PER_STAGE>(); break;
    default: pl::ring_wait_loads<0>(); break;
  }
}
}  // namespace gs_loader

extern "C" __device__ void gs_loader_role_load(const void* params, unsigned variant) {
  (void)variant;
  using namespace gs_loader;
  const GsLoaderParams& p = *static_cast<const GsLoaderParams*>(params);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) - pipelink_gs_warp_load();  // 0: A rows, 1: B^T rows
  const int depth = pipelink_gs_depth();
  unsigned char* ring = pipelink_smem + pipelink_gs_ring() + wave * (GS_TILE_M * 128);
  const int tiles_n = p.n / GS_TILE_N;
  const int row0 = wave == 0 ? (int)(blockIdx.x / tiles_n) * GS_TILE_M : (int)(blockIdx.x % tiles_n) * GS_TILE_N;
  const uint32_t row_pitch = (uint32_t)p.k * 2u;
  const __amdgpu_buffer_rsrc_t rows = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(wave == 0 ? p.a : p.bt), 0,
                                                                        (int)((uint32_t)(wave == 0 ? p.m : p.n) * row_pitch), 0x00020000);
  const int r8 = lane >> 3, pos = lane & 7;
  // rows of one load are 8 consecutive rows starting at a multiple of 8
  const uint32_t lane_offset = (uint32_t)(row0 + r8) * row_pitch + 16u * (uint32_t)(pos ^ r8);
  const int stages = p.k / GS_TILE_K;
  // Stages in flight behind the one being issued.  A stage may only be refilled once it is read, so depth - 1 is the
  // most; one less leaves a free stage between this role and the readers (with none, every fill waits for a hand-shake:
  // measured 2.9 ms against 1.85 ms for the 8192^3 product), and 63 loads per wave cap it at 3.
  const int ahead = depth <= 2 ? 1 : (depth - 2 < 3 ? depth - 2 : 3);
  bool ok = true;
  for (int s = 0; s < stages; ++s) {
    const int slot = s % depth, fill = s / depth;
    // the stage's previous contents have been read by every mma wave
    if (fill > 0) ok &= pl::ring_wait(pl::ring_counter(pipelink_smem, pipelink_gs_empty(), slot), (uint32_t)fill * 4u);
    issue_stage(rows, lane_offset, row_pitch, (uint32_t)s * 128u, ring + slot * GS_STAGE_BYTES);
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
#include "include/gs_abi.h"
#endif

PL_STAGE("gs.loader", "0.1.0");
PL_PARAMS(GsLoaderParams);
PL_ROLE(load, gs_loader_role_load, GS_LOAD_WAVES);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
// ring stage = 256 rows (128 of A, 128 of B^T) x 64 bf16
PL_RING(ab_ring, "produce", load, "bf16", 16, 256, 64, "pipelink_gs_depth", 32768, "pipelink_gs_full", "warps(load)", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_RING("pipelink_gs_ring", "smem", 0, "pipelink_gs_depth", 32768, 1024, "kernel");
PL_CLAIM_RING("pipelink_gs_full", "mbarrier", 0, "pipelink_gs_depth", 1, 1, "kernel");
PL_CLAIM_RING("pipelink_gs_empty", "mbarrier", 0, "pipelink_gs_depth", 1, 1, "kernel");
PL_CLAIM_WARPS("pipelink_gs_warp_load", load, GS_LOAD_WAVES);
PL_USES("pipelink_gs_warp_load");
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_PRELUDE("include/gs_abi.h");
PL_EMIT_MAIN()
