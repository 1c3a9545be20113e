// Package oe.epilogue.wide: the epilogue of the one-epilogue example for the wide matrix package -- per-column scale
// and bias, bf16 store, of one wave's 128 x 64 accumulator.  Same contract as oe.epilogue (the accumulator arrives
// through a function this package declares and the linker generates for the producer's home), but taken one 32 x 32
// block at a time (`<fn>_block`), so that 128 values per lane need not sit in vector registers at once.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/oe_abi.h"

extern "C" __device__ void oe_epilogue_wide_import_acc_ready();
extern "C" __device__ void oe_epilogue_wide_import_acc_block(const void* source, int block, float* dest);  // dest: 16 floats
extern "C" __device__ void oe_epilogue_wide_import_acc_done();

namespace oe_epilogue_wide {
constexpr int FRM = 4, FRN = 2;  // 32 x 32 blocks of the wave's share: rows, columns
__device__ __forceinline__ uint16_t bf16_rne(float x) {
  uint32_t u = __float_as_uint(x);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
}  // namespace oe_epilogue_wide

extern "C" __device__ void oe_epilogue_wide_store(const void* view, const OeTile* tile, const void* source) {
  using namespace oe_epilogue_wide;
  const OeEpilogueParams& p = *static_cast<const OeEpilogueParams*>(static_cast<const pipelink_host_view*>(view)->residue);
  const int lane = threadIdx.x & 63;
  oe_epilogue_wide_import_acc_ready();
#pragma unroll
  for (int j = 0; j < FRN; ++j) {
    const int col = tile->col0 + 32 * j + (lane & 31);
    const float scale = col < p.n ? p.scale[col] : 0.0f, bias = col < p.n ? p.bias[col] : 0.0f;
#pragma unroll
    for (int i = 0; i < FRM; ++i) {
      float acc[16];
      oe_epilogue_wide_import_acc_block(source, i * FRN + j, acc);
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = tile->row0 + 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4;
        if (row < p.m && col < p.n) p.c[(int64_t)row * p.n + col] = bf16_rne(__builtin_fmaf(acc[r], scale, bias));
      }
    }
  }
  oe_epilogue_wide_import_acc_done();
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.epilogue.wide", "0.1.0");
PL_PARAMS(OeEpilogueParams);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_EXPORT(oe_epilogue_wide_store, oe_epilogue_wide_store,
          "extern \"C\" __device__ void oe_epilogue_wide_store(const void* view, const OeTile* tile, const void* source);");
PL_SERVE(epilogue, "oe_epilogue_wide_store");
PL_IMPORT_TENSOR(acc, oe_epilogue_wide_import_acc, "gemm_accumulator", "f32", 128, 64, "mfma32x32c");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
