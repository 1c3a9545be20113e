#pragma once
// Body shared by the three matrix packages of the one-epilogue example.  HOME selects where the wave's
// 64 x 64 fp32 accumulator is when it is handed over: 0 = accumulation registers, 1 = vector registers,
// 2 = a row-major tile in LDS.  Everything else -- the ring protocol, the MFMA loop -- is the matrix role
// of the three-package GEMM example.
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
template <int HOME>
__device__ __forceinline__ void role(const void* params, unsigned char* tile_lds) {
  const OeMmaParams& p = *static_cast<const OeMmaParams*>(params);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)) - pipelink_oe_warp_mma();
  const int depth = pipelink_gs_depth();
  const unsigned char* ring = pipelink_smem + pipelink_gs_ring();
  const int tiles_n = p.n / OE_TILE;
  const OeTile tile{(int)(blockIdx.x / tiles_n) * OE_TILE + 64 * (wave >> 1), (int)(blockIdx.x % tiles_n) * OE_TILE + 64 * (wave & 1)};
  const int arow = 64 * (wave >> 1) + (lane & 31), brow = 64 * (wave & 1) + (lane & 31), half = lane >> 5;
  v16f acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
  const int stages = p.k / OE_TILE_K;
  bool ok = true;
  // Fragment registers are double-buffered by half stages: while the 8 MFMAs of one half (two 16-element sub-steps)
  // run, the 8 reads of the next half are on their way.  Set 0 holds a stage's first half, set 1 its second.
  v8bf fa[2][2][2], fb[2][2][2];
  auto read_half = [&](int s, int set) {
    const int slot = s % depth, use = s / depth;
    if (set == 0) ok &= pl::ring_wait(pl::ring_counter(pipelink_smem, pipelink_gs_full(), slot), ((uint32_t)use + 1u) * OE_LOAD_WAVES);
    const unsigned char* a_rows = ring + slot * OE_STAGE_BYTES;
    const unsigned char* b_rows = a_rows + OE_TILE * 128;
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
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][k2][i], fb[set][k2][j], acc[i][j], 0, 0, 0);
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
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int row = 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4, col = 32 * j + (lane & 31);
          *reinterpret_cast<float*>(tile_lds + row * OE_LDS_PITCH + col * 4) = acc[i][j][r];
        }
    pipelink_call_epilogue(&view, &tile, tile_lds);
  } else {
    // the frame handed over: 64 floats per lane in fragment order, pinned in the home's register class
    float frame[64];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          float v = acc[i][j][r];
          if constexpr (HOME == 0) asm volatile("" : "+a"(v)); else asm volatile("" : "+v"(v));
          frame[(i * 2 + j) * 16 + r] = v;
        }
    pipelink_call_epilogue(&view, &tile, frame);
  }
}
}  // namespace oe_mma
