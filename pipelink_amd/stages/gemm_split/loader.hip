// Package gs.loader: fills the LDS ring of the three-package GEMM example.
//
// One wave.  A ring stage holds 64 contraction elements (128 bytes) of the tile's 128 A rows,
// then of its 128 B^T rows.  One buffer_load_dwordx4 ... lds moves 8 rows: lane i lands at
// byte 16 * i of the 1 KB piece, i.e. row i / 8, 16-byte position i % 8, and fetches the chunk
// that belongs there under the swizzle  position = chunk ^ (row % 8)  the mma role reads with.
// The wave runs one stage ahead: it issues stage s, then waits until the 32 loads of stage
// s - 1 have landed (vmcnt(32)) and arrives on that stage's `full` counter.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <pipelink/ring.hpp>
#include "include/gs_abi.h"

extern "C" __device__ int pipelink_gs_depth();  // ring stages, bound at link time
extern "C" __device__ int pipelink_gs_ring();   // byte offset of the ring in dynamic LDS
extern "C" __device__ int pipelink_gs_full();   // first 16-byte slot of the full counters
extern "C" __device__ int pipelink_gs_empty();  // first 16-byte slot of the empty counters

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace gs_loader {
typedef __attribute__((address_space(3))) void* lds_ptr;
constexpr int LOADS_PER_STAGE = 2 * GS_TILE_M / 8;  // 32

__device__ __forceinline__ void issue_stage(__amdgpu_buffer_rsrc_t a, __amdgpu_buffer_rsrc_t b, uint32_t a_lane,
                                            uint32_t b_lane, uint32_t row_pitch, uint32_t kbyte, unsigned char* stage) {
#pragma unroll
  for (int i = 0; i < GS_TILE_M / 8; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(a, (lds_ptr)(stage + i * 1024), 16, (int)(a_lane + i * 8 * row_pitch), (int)kbyte, 0, 0);
#pragma unroll
  for (int i = 0; i < GS_TILE_N / 8; ++i)
    __builtin_amdgcn_raw_ptr_buffer_load_lds(b, (lds_ptr)(stage + GS_TILE_M * 128 + i * 1024), 16,
                                             (int)(b_lane + i * 8 * row_pitch), (int)kbyte, 0, 0);
}
}  // namespace gs_loader

extern "C" __device__ void gs_loader_role_load(const void* params, unsigned variant) {
  (void)variant;
  using namespace gs_loader;
  const GsLoaderParams& p = *static_cast<const GsLoaderParams*>(params);
  const int lane = threadIdx.x & 63;
  const int depth = pipelink_gs_depth();
  unsigned char* ring = pipelink_smem + pipelink_gs_ring();
  const int tiles_n = p.n / GS_TILE_N;
  const int row0 = (blockIdx.x / tiles_n) * GS_TILE_M, col0 = (blockIdx.x % tiles_n) * GS_TILE_N;
  const uint32_t row_pitch = (uint32_t)p.k * 2u;
  const __amdgpu_buffer_rsrc_t a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.a), 0, (int)((uint32_t)p.m * row_pitch), 0x00020000);
  const __amdgpu_buffer_rsrc_t b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.bt), 0, (int)((uint32_t)p.n * row_pitch), 0x00020000);
  const int r8 = lane >> 3, pos = lane & 7;
  const uint32_t chunk = 16u * (uint32_t)(pos ^ r8);  // rows of one load are 8 consecutive rows starting at a multiple of 8
  const uint32_t a_lane = (uint32_t)(row0 + r8) * row_pitch + chunk;
  const uint32_t b_lane = (uint32_t)(col0 + r8) * row_pitch + chunk;
  const int stages = p.k / GS_TILE_K;
  bool ok = true;
  for (int s = 0; s < stages; ++s) {
    const int slot = s % depth, fill = s / depth;
    // the stage's previous contents have been read by every mma wave
    if (fill > 0) ok &= pl::ring_wait(pl::ring_counter(pipelink_smem, pipelink_gs_empty(), slot), (uint32_t)fill * 4u);
    issue_stage(a, b, a_lane, b_lane, row_pitch, (uint32_t)s * 128u, ring + slot * GS_STAGE_BYTES);
    if (s > 0) {
      pl::ring_wait_loads<LOADS_PER_STAGE>();  // everything but the stage just issued has landed
      if (lane == 0) pl::ring_arrive(pl::ring_counter(pipelink_smem, pipelink_gs_full(), (s - 1) % depth));
    }
  }
  pl::ring_wait_loads<0>();
  if (lane == 0) {
    pl::ring_arrive(pl::ring_counter(pipelink_smem, pipelink_gs_full(), (stages - 1) % depth));
    if (!ok) atomicOr(p.status, 1u);
  }
}
#else
#include "include/gs_abi.h"
#endif

PL_STAGE("gs.loader", "0.1.0");
PL_PARAMS(GsLoaderParams);
PL_ROLE(load, gs_loader_role_load, 1);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
// ring stage = 256 rows (128 of A, 128 of B^T) x 64 bf16
PL_RING(ab_ring, "produce", load, "bf16", 16, 256, 64, "pipelink_gs_depth", 32768, "pipelink_gs_full", "1", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_RING("pipelink_gs_ring", "smem", 0, "pipelink_gs_depth", 32768, 1024, "kernel");
PL_CLAIM_RING("pipelink_gs_full", "mbarrier", 0, "pipelink_gs_depth", 1, 1, "kernel");
PL_CLAIM_RING("pipelink_gs_empty", "mbarrier", 0, "pipelink_gs_depth", 1, 1, "kernel");
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_PRELUDE("include/gs_abi.h");
PL_EMIT_MAIN()
