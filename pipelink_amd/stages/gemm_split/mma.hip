// Package gs.mma: the matrix role of the three-package GEMM example.
//
// Four waves as 2 (rows) x 2 (columns), 64 x 64 outputs each = 2 x 2 accumulators of
// v_mfma_f32_32x32x16_bf16.  Per ring stage (64 contraction elements) a wave waits for the
// stage's `full` count (one arrival per loader wave), reads its two A fragments and two B fragments for
// each of the four 16-element sub-steps from LDS, half a stage at a time into one of two register sets (the
// reads of one half are on their way while the other half is multiplied), and says on `empty` that it has
// read the stage.
// At the end it hands the accumulator to whoever serves the `epilogue` channel.
//
// MFMA 32x32x16 bf16 operand of lane l: row l % 32, contraction elements 8 * (l / 32) .. + 8 of
// the sub-step, 16 bytes; a row's 16-byte chunks are stored at position chunk ^ (row % 8).
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <pipelink/ring.hpp>
#include "include/gs_abi.h"

extern "C" __device__ int pipelink_gs_depth();
extern "C" __device__ int pipelink_gs_ring();
extern "C" __device__ int pipelink_gs_full();
extern "C" __device__ int pipelink_gs_empty();
extern "C" __device__ int pipelink_gs_warp_mma();  // index of this role's first wave in the workgroup

extern "C" __device__ void pipelink_call_epilogue(const void* view, const GsTile* tile, const GsAcc* acc, int wave);

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace gs_mma {
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ v8bf read_frag(const unsigned char* rows, int row, int chunk) {
  const v4i raw = *reinterpret_cast<const v4i*>(rows + row * 128 + 16 * (chunk ^ (row & 7)));
  return __builtin_bit_cast(v8bf, raw);
}
}  // namespace gs_mma

extern "C" __device__ void gs_mma_role_mma(const void* params, unsigned variant) {
  (void)variant;
  using namespace gs_mma;
  const GsMmaParams& p = *static_cast<const GsMmaParams*>(params);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) - pipelink_gs_warp_mma();
  const int depth = pipelink_gs_depth();
  const unsigned char* ring = pipelink_smem + pipelink_gs_ring();
  const int tiles_n = p.n / GS_TILE_N;
  const GsTile tile{(int)(blockIdx.x / tiles_n) * GS_TILE_M, (int)(blockIdx.x % tiles_n) * GS_TILE_N};
  const int arow = 64 * (wave >> 1) + (lane & 31);  // + 32 * i: this lane's A row in the stage
  const int brow = 64 * (wave & 1) + (lane & 31);   // + 32 * j
  const int half = lane >> 5;
  GsAcc acc;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc.v[i][j][r] = 0.0f;
  const int stages = p.k / GS_TILE_K;
  bool ok = true;
  // Fragment registers are double-buffered by half stages: while the 8 MFMAs of one half (two 16-element sub-steps)
  // run, the 8 reads of the next half are on their way.  Set 0 holds a stage's first half, set 1 its second.
  v8bf fa[2][2][2], fb[2][2][2];
  auto read_half = [&](int s, int set) {
    const int slot = s % depth, use = s / depth;
    if (set == 0) ok &= pl::ring_wait(pl::ring_counter(pipelink_smem, pipelink_gs_full(), slot), ((uint32_t)use + 1u) * GS_LOAD_WAVES);
    const unsigned char* a_rows = ring + slot * GS_STAGE_BYTES;
    const unsigned char* b_rows = a_rows + GS_TILE_M * 128;
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        fa[set][k2][i] = read_frag(a_rows, arow + 32 * i, 2 * (2 * set + k2) + half);
        fb[set][k2][i] = read_frag(b_rows, brow + 32 * i, 2 * (2 * set + k2) + half);
      }
  };
  auto multiply = [&](int set) {
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc.v[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][k2][i], fb[set][k2][j], acc.v[i][j], 0, 0, 0);
  };
  read_half(0, 0);
  for (int s = 0; s < stages; ++s) {
    read_half(s, 1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(0);
    __builtin_amdgcn_sched_barrier(0);
    pl::ring_wait_reads();  // both halves of stage s are in registers
    if (lane == 0) pl::ring_arrive(pl::ring_counter(pipelink_smem, pipelink_gs_empty(), s % depth));
    if (s + 1 < stages) read_half(s + 1, 0);
    __builtin_amdgcn_sched_barrier(0);
    multiply(1);
    __builtin_amdgcn_sched_barrier(0);
  }
  if (!ok && lane == 0) atomicOr(p.status, 2u);
  const pipelink_host_view view{params, nullptr};
  pipelink_call_epilogue(&view, &tile, &acc, wave);
}
#else
#include "include/gs_abi.h"
#endif

PL_STAGE("gs.mma", "0.1.0");
PL_PARAMS(GsMmaParams);
PL_ROLE(mma, gs_mma_role_mma, 4);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_RING(ab_ring, "consume", mma, "bf16", 16, 256, 64, "pipelink_gs_depth", 32768, "pipelink_gs_full", "warps(load)", load,
        "pipelink_gs_empty", "warps(mma)", mma, load);
PL_CLAIM_WARPS("pipelink_gs_warp_mma", mma, 4);
PL_CALL(epilogue, "gs_epilogue_store",
        "extern \"C\" __device__ void pipelink_call_epilogue(const void* view, const GsTile* tile, const GsAcc* acc, int wave);");
PL_USES("pipelink_gs_depth");
PL_USES("pipelink_gs_ring");
PL_USES("pipelink_gs_full");
PL_USES("pipelink_gs_empty");
PL_USES("pipelink_gs_warp_mma");
PL_PRELUDE("include/gs_abi.h");
PL_EMIT_MAIN()
