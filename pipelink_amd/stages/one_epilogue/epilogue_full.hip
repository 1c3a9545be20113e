// Package oe.epilogue.full: the epilogue of the one-epilogue example for the 256 x 256 matrix package -- per-column
// scale and bias, bf16 store, of one wave's 128 x 128 accumulator.  Same contract as oe.epilogue (the accumulator
// arrives through a function this package declares and the linker generates for the producer's home), taken one
// 32 x 32 block at a time so that 256 values per lane need not sit in vector registers at once.  The producer hands
// over the TRANSPOSE of its share of C: tensor rows are output columns, tensor columns output rows, so a lane's four
// consecutive tensor rows of a block are four consecutive bf16 of one output row: one 8-byte store, and the two lanes
// l and l + 32 together write 16 contiguous bytes.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/oe_abi.h"

extern "C" __device__ void oe_epilogue_full_import_acc_ready();
extern "C" __device__ void oe_epilogue_full_import_acc_block(const void* source, int block, float* dest);  // dest: 16 floats
extern "C" __device__ void oe_epilogue_full_import_acc_done();

namespace oe_epilogue_full {
constexpr int FR = 4;  // 32 x 32 blocks of the wave's share, either way
typedef float v4f __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // nearest even
}
}  // namespace oe_epilogue_full

// tile->row0: the share's first output column; tile->col0: its first output row
extern "C" __device__ void oe_epilogue_full_store(const void* view, const OeTile* tile, const void* source) {
  using namespace oe_epilogue_full;
  const OeEpilogueParams& p = *static_cast<const OeEpilogueParams*>(static_cast<const pipelink_host_view*>(view)->residue);
  const int lane = threadIdx.x & 63;
  oe_epilogue_full_import_acc_ready();
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
      const int row = tile->col0 + 32 * j + (lane & 31);
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = tile->row0 + 32 * i + 8 * q + 4 * (lane >> 5);
        uint2 out;
        out.x = pack_bf16x2(__builtin_fmaf(acc[4 * q + 0], scale[q].x, bias[q].x), __builtin_fmaf(acc[4 * q + 1], scale[q].y, bias[q].y));
        out.y = pack_bf16x2(__builtin_fmaf(acc[4 * q + 2], scale[q].z, bias[q].z), __builtin_fmaf(acc[4 * q + 3], scale[q].w, bias[q].w));
        *reinterpret_cast<uint2*>(p.c + (int64_t)row * p.n + col) = out;
      }
    }
  }
  oe_epilogue_full_import_acc_done();
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
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
