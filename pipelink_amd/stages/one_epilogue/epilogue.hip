// Package oe.epilogue: per-column scale and bias, bf16 store, of one wave's 64 x 64 accumulator --
// wherever the matrix package it is linked against keeps it.  The accumulator arrives through
// oe_epilogue_import_acc, which this package declares and the linker generates for the producer's home;
// this source is the same for all three producers.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/oe_abi.h"

extern "C" __device__ void oe_epilogue_import_acc_ready();
extern "C" __device__ void oe_epilogue_import_acc(const void* source, float* dest);  // dest: 64 floats, fragment order
extern "C" __device__ void oe_epilogue_import_acc_done();

namespace oe_epilogue {
__device__ __forceinline__ uint16_t bf16_rne(float x) {
  uint32_t u = __float_as_uint(x);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
}  // namespace oe_epilogue

extern "C" __device__ void oe_epilogue_store(const void* view, const OeTile* tile, const void* source) {
  const OeEpilogueParams& p = *static_cast<const OeEpilogueParams*>(static_cast<const pipelink_host_view*>(view)->residue);
  const int lane = threadIdx.x & 63;
  float acc[64];
  oe_epilogue_import_acc_ready();
  oe_epilogue_import_acc(source, acc);
  oe_epilogue_import_acc_done();
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = tile->col0 + 32 * j + (lane & 31);
    const float scale = col < p.n ? p.scale[col] : 0.0f, bias = col < p.n ? p.bias[col] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = tile->row0 + 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4;
        if (row < p.m && col < p.n)
          p.c[(int64_t)row * p.n + col] = oe_epilogue::bf16_rne(__builtin_fmaf(acc[(i * 2 + j) * 16 + r], scale, bias));
      }
  }
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.epilogue", "0.1.0");
PL_PARAMS(OeEpilogueParams);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_EXPORT(oe_epilogue_store, oe_epilogue_store,
          "extern \"C\" __device__ void oe_epilogue_store(const void* view, const OeTile* tile, const void* source);");
PL_SERVE(epilogue, "oe_epilogue_store");
PL_IMPORT_TENSOR(acc, oe_epilogue_import_acc, "gemm_accumulator", "f32", 64, 64, "mfma32x32c");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
