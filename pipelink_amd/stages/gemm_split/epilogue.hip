// Package gs.epilogue: bias + GELU + bf16 store of one mma wave's accumulator.
//
// GELU(x) = x * (1 + erf(x / sqrt 2)) / 2 (the erf form, torch's default).  erf is evaluated
// with the rational approximation of Abramowitz & Stegun 7.1.26 (absolute error below 1.5e-7,
// far inside the bf16 rounding of the result) on the hardware exp2 and reciprocal, so the
// package needs no device library.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/gs_abi.h"

namespace gs_epilogue {
__device__ __forceinline__ float erf_as(float x) {
  const float ax = __builtin_fabsf(x);
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * ax);
  const float poly = t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
  const float e = __builtin_amdgcn_exp2f(-ax * ax * 1.4426950408889634f);
  const float y = 1.0f - poly * e;
  return x < 0.0f ? -y : y;
}
__device__ __forceinline__ float gelu(float x) { return 0.5f * x * (1.0f + erf_as(x * 0.70710678118654752f)); }
__device__ __forceinline__ uint16_t bf16_rne(float x) {
  uint32_t u = __float_as_uint(x);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
}  // namespace gs_epilogue

extern "C" __device__ void gs_epilogue_store(const void* view, const GsTile* tile, const GsAcc* acc, int wave) {
  using namespace gs_epilogue;
  const GsEpilogueParams& p = *static_cast<const GsEpilogueParams*>(static_cast<const pipelink_host_view*>(view)->residue);
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int col = tile->col0 + 64 * (wave & 1) + 32 * j + (lane & 31);
    const float bias = col < p.n ? p.bias[col] : 0.0f;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = tile->row0 + 64 * (wave >> 1) + 32 * i + 8 * (r / 4) + 4 * (lane >> 5) + r % 4;
        if (row < p.m && col < p.n) p.c[(int64_t)row * p.n + col] = bf16_rne(gelu(acc->v[i][j][r] + bias));
      }
  }
}
#else
#include "include/gs_abi.h"
#endif

PL_STAGE("gs.epilogue", "0.1.0");
PL_PARAMS(GsEpilogueParams);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_EXPORT(gs_epilogue_store, gs_epilogue_store,
          "extern \"C\" __device__ void gs_epilogue_store(const void* view, const GsTile* tile, const GsAcc* acc, int wave);");
PL_SERVE(epilogue, "gs_epilogue_store");
PL_PRELUDE("include/gs_abi.h");
PL_EMIT_MAIN()
