#pragma once
// Body shared by the matrix packages of the one-epilogue example.  HOME selects where the wave's fp32
// accumulator is when it is handed over: 0 = accumulation registers, 1 = vector registers, 2 = a row-major
// tile in LDS.  FRM x FRN is the wave's share in 32 x 32 fragments: 2 x 2 (a 64 x 64 share of a 128 x 128
// workgroup tile, the three homes) or 4 x 2 (128 x 64 of 256 x 128: 128 accumulation registers, which with the
// operand registers is what a wave may have while loader waves share its SIMD; a quarter fewer operand bytes per
// flop through L2 and LDS, and stages half as large again in flight).  Everything else -- the ring protocol,
// the MFMA loop -- is the matrix role of the three-package GEMM example.
#include <pipelink/ring.hpp>
#include "include/oe_abi.h"

extern "C" __device__ int pipelink_gs_depth();
extern "C" __device__ int pipelink_gs_ring();
extern "C" __device__ int pipelink_gs_full();
extern "C" __device__ int pipelink_gs_empty();
extern "C" __device__ int pipelink_oe_warp_mma();
extern "C" __device__ void pipelink_call_epilogue(const void* view, const OeTile* tile, const void* source);

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace oe_mma {
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ __forceinline__ v8bf read_frag(const unsigned char* rows, int row, int chunk) {
  const v4i raw = *reinterpret_cast<const v4i*>(rows + row * 128 + 16 * (chunk ^ (row & 7)));
  return __builtin_bit_cast(v8bf, raw);
}

// `tile_lds` is the wave's LDS tile for HOME 2 (unused otherwise)
template <int HOME, int FRM = 2, int FRN = 2>
__device__ __forceinline__ void role(const void* params, unsigned char* tile_lds) {
  constexpr int WTM = 32 * FRM, WTN = 32 * FRN;      // the wave's share: rows, columns
  constexpr int TILE_M = 2 * WTM, TILE_N = 2 * WTN;  // the workgroup's tile: 2 x 2 waves
  constexpr int STAGE_BYTES = (TILE_M + TILE_N) * 128;  // A rows then B^T rows, 64 bf16 each
  constexpr int LOAD_WAVES = FRM == 2 ? OE_LOAD_WAVES : OE_WIDE_LOAD_WAVES;
  static_assert(HOME == 0 || (FRM == 2 && FRN == 2), "the larger share is handed over in accumulation registers");
  const OeMmaParams& p = *static_cast<const OeMmaParams*>(params);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) - pipelink_oe_warp_mma();
  const int depth = pipelink_gs_depth();
  const unsigned char* ring = pipelink_smem + pipelink_gs_ring();
  const int tiles_n = p.n / TILE_N;
  const OeTile tile{(int)(blockIdx.x / tiles_n) * TILE_M + WTM * (wave >> 1), (int)(blockIdx.x % tiles_n) * TILE_N + WTN * (wave & 1)};
  const int arow = WTM * (wave >> 1) + (lane & 31), brow = WTN * (wave & 1) + (lane & 31), half = lane >> 5;
  v16f acc[FRM][FRN];
#pragma unroll
  for (int i = 0; i < FRM; ++i)
#pragma unroll
    for (int j = 0; j < FRN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const int stages = p.k / OE_TILE_K;
  bool ok = true;
  // Fragment registers are double-buffered by half stages: while the 8 MFMAs of one half (two 16-element sub-steps)
  // run, the 8 reads of the next half are on their way.  Set 0 holds a stage's first half, set 1 its second.
  v8bf fa[2][2][FRM], fb[2][2][FRN];
  auto read_half = [&](int s, int set) {
    const int slot = s % depth, use = s / depth;
    if (set == 0) ok &= pl::ring_wait(pl::ring_counter(pipelink_smem, pipelink_gs_full(), slot), ((uint32_t)use + 1u) * LOAD_WAVES);
    const unsigned char* a_rows = ring + slot * STAGE_BYTES;
    const unsigned char* b_rows = a_rows + TILE_M * 128;
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2) {
#pragma unroll
      for (int i = 0; i < FRM; ++i) fa[set][k2][i] = read_frag(a_rows, arow + 32 * i, 2 * (2 * set + k2) + half);
#pragma unroll
      for (int j = 0; j < FRN; ++j) fb[set][k2][j] = read_frag(b_rows, brow + 32 * j, 2 * (2 * set + k2) + half);
    }
  };
  auto multiply = [&](int set) {
#pragma unroll
    for (int k2 = 0; k2 < 2; ++k2)
#pragma unroll
      for (int i = 0; i < FRM; ++i)
#pragma unroll
        for (int j = 0; j < FRN; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][k2][i], fb[set][k2][j], acc[i][j], 0, 0, 0);
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
  if constexpr (HOME == 2) {
    // row-major fp32 tile, rows OE_LDS_PITCH bytes apart
#pragma unroll
    for (int i = 0; i < FRM; ++i)
#pragma unroll
      for (int j = 0; j < FRN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, col = 32 * j + (lane & 31);
          *reinterpret_cast<float*>(tile_lds + row * OE_LDS_PITCH + col * 4) = acc[i][j][r];
        }
    pipelink_call_epilogue(&view, &tile, tile_lds);
  } else {
    // the frame handed over: 16 floats per fragment and lane in fragment order, pinned in the home's register class
    float frame[FRM * FRN * 16];
#pragma unroll
    for (int i = 0; i < FRM; ++i)
#pragma unroll
      for (int j = 0; j < FRN; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = acc[i][j][r];
          if constexpr (HOME == 0) asm volatile("" : "+a"(v)); else asm volatile("" : "+v"(v));
          frame[(i * FRN + j) * 16 + r] = v;
        }
    pipelink_call_epilogue(&view, &tile, frame);
  }
}
}  // namespace oe_mma
