// Device-side helpers shared by the MoK stage sources: vector types, the MFMA wrapper and
// the contract that says where one element of the grouped-GEMM accumulator lives.
#ifndef PIPELINK_MOK_DEVICE_HPP
#define PIPELINK_MOK_DEVICE_HPP

#include <hip/hip_runtime.h>
#include <stdint.h>
#include "mok_abi.h"

namespace mok {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));

// ---- tile geometry published by the GEMM owner (facts mok.gemm.*) -------------------
// One workgroup tile = TILE_X routed rows x TILE_W weight rows, 4 waves (one per SIMD) as
// 2 (rows) x 2 (weights), each wave a 128 x 128 sub-tile.  For the gate/up op the weight
// rows are TILE_W/2 gate columns followed by the same TILE_W/2 up columns, so gate and up of
// one output element meet in one lane.
constexpr int TILE_X = 256;
constexpr int TILE_W = 256;
constexpr int K_SLOT = 64;      // contraction bytes per ring slot = one MFMA 32x32x64 step
constexpr int K_PAIR = 128;     // contraction bytes one dword of four e8m0 block scales covers
constexpr int WFRAGS = 4;       // 32-row weight fragments per wave
constexpr int XFRAGS = 4;       // 32-row activation fragments per wave
constexpr int THREADS = 256;
constexpr int BUF_BYTES = TILE_X * K_SLOT;                // one ring buffer: 256 rows x 64 bytes (TILE_W == TILE_X)
constexpr int WSCALE_BYTES = 4 * TILE_W * 4;             // four buffers of one dword (4 block scales) per weight row
constexpr int XSCALE_BYTES = 2 * TILE_X * 16;            // two buffers of 16 scale bytes (8 slots) per routed row

// fp32 accumulator of one wave: [weight fragment][row fragment] MFMA 32x32 C tiles.
// Element (reg r, lane l) of tile (a, b) is
//   weight row  = wrow0(a) + 8*(r/4) + 4*(l/32) + r%4      (output column)
//   routed row  = xrow0(b) + l%32
// with wrow0/xrow0 below.  This is the placement the activation owner imports.
struct AccFrag {
  v16f v[WFRAGS][XFRAGS];
};

// One fragment of the accumulator, which stays in the accumulator registers up to here.  An epilogue takes each
// fragment through this where it starts to use it: the compiler may otherwise copy the whole tile to vector
// registers as soon as the mainloop is over, ahead of the next tile's prefetch, which leaves that code short of
// registers (its spills then wait for the prefetch's loads, because every wait on a scratch load does).
__device__ __forceinline__ v16f from_acc(v16f v) {
  asm volatile("" : "+a"(v));
  return v;
}

// What the GEMM owner's prefetch export hands to its forward export for the same tile: the
// lane's gathered routed-row offsets (they cost a dependent global load, which the prefetch
// takes off the forward call's critical path).  Opaque to the other stages.
struct GemmCarry {
  uint32_t xsrc[TILE_X / 16 / (THREADS / 64)];
  uint32_t xscsrc;
};

__device__ __forceinline__ int wave_w(int wave) { return wave & 1; }
__device__ __forceinline__ int wave_x(int wave) { return wave >> 1; }
// first tile-local weight row of fragment a for this wave (rows [0,128) | [128,256))
__device__ __forceinline__ int wrow0(int wave, int a) {
  return (a < 2 ? 0 : TILE_W / 2) + wave_w(wave) * 64 + (a & 1) * 32;
}
__device__ __forceinline__ int xrow0(int wave, int b) { return wave_x(wave) * 128 + b * 32; }

typedef __attribute__((address_space(3))) void* lptr_t;

// threadIdx.x as a value the compiler cannot merge with an earlier copy: code that runs after
// a register-hungry loop derives its lane indices from this, so they are computed where they
// are used instead of being kept (spilled) across the loop.
__device__ __forceinline__ int fresh_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

}  // namespace mok

#endif
