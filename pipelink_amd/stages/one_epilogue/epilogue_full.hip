// Package oe.epilogue.full: the epilogue of the one-epilogue example for the 256 x 256 matrix package -- per-column
// scale and bias, bf16 store, of one wave's 128 x 128 accumulator.  Same contract as oe.epilogue (the accumulator
// arrives through a function this package declares and the linker generates for the producer's home), taken one
// 32 x 32 block at a time so that 256 values per lane need not sit in vector registers at once.  The producer hands
// over the TRANSPOSE of its share of C: tensor rows are output columns, tensor columns output rows, so a lane's four
// consecutive tensor rows of a block are four consecutive bf16 of one output row.  Stored from the registers that
// would be 8 bytes per lane and 32 rows per instruction (5.7 % of the 8192^3 product's time); instead the four waves
// put the workgroup's 256 x 256 bf16 tile together in the matrix package's LDS ring, which is idle by then, and write
// it out 16 bytes per lane, an instruction covering two whole 512-byte rows of the tile.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/oe_abi.h"

extern "C" __device__ int pipelink_oe_full_ring();  // the matrix package's LDS ring: 160 KB, free once every wave has left its loop
extern "C" __device__ void oe_epilogue_full_import_acc_ready();
extern "C" __device__ void oe_epilogue_full_import_acc_block(const void* source, int block, float* dest);  // dest: 16 floats
extern "C" __device__ void oe_epilogue_full_import_acc_done();

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace oe_epilogue_full {
constexpr int FR = 4;  // 32 x 32 blocks of the wave's share, either way
constexpr int PITCH = OE_FULL_TILE * 2 + 16;  // bytes between rows of the staged tile: lanes of one write spread over all banks
static_assert(OE_FULL_TILE * PITCH <= 2 * OE_FULL_BUFFERS * OE_FULL_TILE * 64, "the staged tile must fit the ring");
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // nearest even
}
}  // namespace oe_epilogue_full

// tile->row0: the share's first output column; tile->col0: its first output row.  Every wave of the workgroup calls
// this once (it holds two workgroup barriers).
extern "C" __device__ void oe_epilogue_full_store(const void* view, const OeTile* tile, const void* source) {
  using namespace oe_epilogue_full;
  const OeEpilogueParams& p = *static_cast<const OeEpilogueParams*>(static_cast<const pipelink_host_view*>(view)->residue);
  const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  unsigned char* stage = pipelink_smem + pipelink_oe_full_ring();
  const int n0 = tile->row0 & ~(OE_FULL_TILE - 1), m0 = tile->col0 & ~(OE_FULL_TILE - 1);  // the workgroup's tile
  const int nw = tile->row0 - n0, mw = tile->col0 - m0;                                    // the wave's share inside it
  oe_epilogue_full_import_acc_ready();
  __syncthreads();  // every wave has read its last operands: the ring is free
#pragma unroll
  for (int i = 0; i < FR; ++i) {      // 32 output columns
    v4f scale[4], bias[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int col = tile->row0 + 32 * i + 8 * q + 4 * (lane >> 5);  // multiple of 4; N is a multiple of 256
      scale[q] = *reinterpret_cast<const v4f*>(p.scale + col);
      bias[q] = *reinterpret_cast<const v4f*>(p.bias + col);
    }
#pragma unroll
    for (int j = 0; j < FR; ++j) {    // 32 output rows
      float acc[16];
      oe_epilogue_full_import_acc_block(source, i * FR + j, acc);
      unsigned char* row = stage + (mw + 32 * j + (lane & 31)) * PITCH + (nw + 32 * i + 4 * (lane >> 5)) * 2;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        uint2 out;
        out.x = pack_bf16x2(__builtin_fmaf(acc[4 * q + 0], scale[q].x, bias[q].x), __builtin_fmaf(acc[4 * q + 1], scale[q].y, bias[q].y));
        out.y = pack_bf16x2(__builtin_fmaf(acc[4 * q + 2], scale[q].z, bias[q].z), __builtin_fmaf(acc[4 * q + 3], scale[q].w, bias[q].w));
        *reinterpret_cast<uint2*>(row + 16 * q) = out;
      }
    }
  }
  oe_epilogue_full_import_acc_done();
  __syncthreads();  // the tile is whole
  // wave w writes rows 64 w .. 64 w + 63 of the tile: lanes 0-31 one row, lanes 32-63 the next, 16 bytes each
#pragma unroll 4
  for (int it = 0; it < OE_FULL_TILE / 4 / 2; ++it) {
    const int r = 64 * wave + 2 * it + (lane >> 5), c16 = lane & 31;
    const v4i piece = *reinterpret_cast<const v4i*>(stage + r * PITCH + 16 * c16);
    *reinterpret_cast<v4i*>(p.c + (int64_t)(m0 + r) * p.n + n0 + 8 * c16) = piece;
  }
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.epilogue.full", "0.1.0");
PL_PARAMS(OeEpilogueParams);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_EXPORT(oe_epilogue_full_store, oe_epilogue_full_store,
          "extern \"C\" __device__ void oe_epilogue_full_store(const void* view, const OeTile* tile, const void* source);");
PL_SERVE(epilogue, "oe_epilogue_full_store");
PL_IMPORT_TENSOR(acc, oe_epilogue_full_import_acc, "gemm_accumulator_transposed", "f32", 128, 128, "mfma32x32c");
PL_USES("pipelink_oe_full_ring");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
