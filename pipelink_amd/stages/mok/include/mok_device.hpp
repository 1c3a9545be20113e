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

// ---- tiles with little to multiply ------------------------------------------------------------------------------
// A tile that holds at most 64 routed rows (the rows an expert has past its last full tile), or at most 64 output
// columns per weight matrix (the columns past the last full column tile), is multiplied in another placement: every
// wave takes 64 routed rows and up to four 32-row weight fragments, in the accumulator's fragments [a][b] with b < 2.
//   SMALL_ROWS: all four waves share routed rows 0..63; wave w owns weight fragments a = 0 and a = 2, tile rows
//               32 w and 128 + 32 w (for the gate/up op: 32 gate columns and the same 32 up columns).
//   SMALL_COLS: wave w owns routed rows 64 w .. 64 w + 63; the weight fragments are tile rows 0, 32 (a = 0, 1) and,
//               for the gate/up op, 128, 160 (a = 2, 3): 64 gate columns and the same 64 up columns.
// Element (reg r, lane l) of fragment (a, b) is weight row wr[a] + 8 (r / 4) + 4 (l / 32) + r % 4, routed row
// xr0 + 32 b + l % 32.  Which placement a tile has follows from its extent alone, so every owner works it out for itself.
enum { TILE_FULL = 0, TILE_SMALL_ROWS = 1, TILE_SMALL_COLS = 2 };
constexpr int SMALL_EXTENT = 64;
// rows: routed rows of the tile that exist; cols: output columns (per weight matrix) from the tile's first that exist
__device__ __forceinline__ int tile_placement(int rows, int cols) {
  return rows <= SMALL_EXTENT ? TILE_SMALL_ROWS : cols <= SMALL_EXTENT ? TILE_SMALL_COLS : TILE_FULL;
}
struct SmallPlacement {
  int xr0;    // first tile-local routed row of the wave
  int wr[4];  // tile-local weight row of fragment a
};
__device__ __forceinline__ SmallPlacement small_placement(int placement, int wave) {
  SmallPlacement p;
  const bool rows = placement == TILE_SMALL_ROWS;
  p.xr0 = rows ? 0 : 64 * wave;
  p.wr[0] = rows ? 32 * wave : 0;
  p.wr[1] = 32;
  p.wr[2] = TILE_W / 2 + (rows ? 32 * wave : 0);
  p.wr[3] = TILE_W / 2 + 32;
  return p;
}
// the fragments a that are multiplied, as a bit mask: a = 0 and 2 for few rows; 0, 1 and (gate/up op) 2, 3 for few columns
constexpr int SMALL_ROWS_FRAGS = 0b0101, SMALL_COLS_FRAGS_GATE_UP = 0b1111, SMALL_COLS_FRAGS_DOWN = 0b0011;

typedef __attribute__((address_space(3))) void* lptr_t;

// Workgroup barrier that orders the workgroup's LDS traffic and nothing else: every LDS access this wave has issued
// has completed (lgkmcnt(0)); vector-memory operations stay in flight.  __syncthreads() also waits for every
// outstanding global -> LDS load and every store.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

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
