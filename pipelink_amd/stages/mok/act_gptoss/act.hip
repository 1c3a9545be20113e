// Owner package mok.act (GPT-OSS flavour): clamped SwiGLU with alpha = 1.702 applied to
// the gate/up accumulator of one tile, rounded to bf16, then requantised to MXFP8 along
// the d_ff axis (one e8m0 scale per 32 columns of a routed row).
//
// Replaces swiglu_fwd_kernel<false, IS_CLAMPED> of
// campaigns/mok/port/act_gptoss/swiglu.cuh:45-217 (MXFP8 branch :157-195).  Differences by
// design: the inputs arrive as fp32 MFMA accumulators instead of bf16 tiles read back
// from HBM, and only the row-wise (forward) quantised copy is written.
//
// The body only uses the placement contract of mok::AccFrag (which routed row and column
// a (fragment, register, lane) triple is); it does not care whether the GEMM owner kept
// the accumulator in AGPRs, VGPRs or LDS.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "../include/mok_device.hpp"

extern "C" __device__ int pipelink_mok_clamp();  // link-time variant: 1 = clamp to +-limit

namespace mok_act_owner {
using namespace mok;

constexpr float SWIGLU_ALPHA = 1.702f;  // campaigns/mok/port/act_gptoss/swiglu.cuh:2

template <bool CLAMPED>
__device__ __forceinline__ float swiglu(float gate, float up, float limit) {
  if (CLAMPED) {
    gate = fminf(gate, limit);
    up = fminf(fmaxf(up, -limit), limit);
  }
  // (up + 1) * gate * sigmoid(alpha * gate), fast exp and reciprocal as in the reference's
  // --use_fast_math build (campaigns/mok/port/build.py:26)
  const float den = 1.0f + __expf(-SWIGLU_ALPHA * gate);
  return (up + 1.0f) * (gate * __builtin_amdgcn_rcpf(den));
}

// e4m3 (OCP) pack of four floats already scaled into [-448, 448]
__device__ __forceinline__ uint32_t pack_e4m3x4(float a, float b, float c, float d) {
  int v = 0;
  v = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, v, false);
  v = __builtin_amdgcn_cvt_pk_fp8_f32(c, d, v, true);
  return (uint32_t)v;
}

template <bool CLAMPED>
__device__ __forceinline__ void forward(const MokActResidue& p, const MokActTask& t, const AccFrag& acc) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int half = lane >> 5;
#pragma unroll
  for (int a = 0; a < 2; ++a) {  // gate fragments a, up fragments a + 2: same rows, same columns
    const int col0 = t.col_begin + wrow0(wave, a);  // 32-column block of d_ff
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b) {
      const int row = t.row_begin + xrow0(wave, b) + (lane & 31);
      float h[16];
      float amax = 0.0f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        h[r] = bf16_round(swiglu<CLAMPED>(acc.v[a][b][r], acc.v[a + 2][b][r], p.swiglu_limit));
        amax = fmaxf(amax, fabsf(h[r]));
      }
      // the other 16 columns of this row's block live in lane ^ 32
      amax = fmaxf(amax, __shfl_xor(amax, 32));
      int e = (int)((__float_as_uint(amax) >> 23) & 0xFFu) - 8;  // floor(log2(amax)) - 8 + 127
      e = e < 0 ? 0 : e;                                          // amax < 2^-118: scale byte 0
      const float inv = __uint_as_float((uint32_t)(254 - e) << 23);  // 2^(127 - e), e <= 247
      const bool live = row < t.row_end && col0 < p.cols;
      if (live) {
        uint8_t* qrow = p.hidden_q + (int64_t)row * p.ld_q + col0 + 4 * half;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          float s[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) s[j] = fminf(fmaxf(h[4 * q + j] * inv, -448.0f), 448.0f);
          *reinterpret_cast<uint32_t*>(qrow + 8 * q) = pack_e4m3x4(s[0], s[1], s[2], s[3]);
        }
        if (half == 0) p.hidden_sc[(int64_t)row * p.ld_sc + (col0 >> 5)] = (uint8_t)e;
      }
    }
  }
}

}  // namespace mok_act_owner

extern "C" __device__ void mok_act_init(const void* view) { (void)view; }

extern "C" __device__ void mok_act_fwd(const void* view, const MokActTask* task, const MokCounters* counters,
                                       uint32_t* phase, const mok::AccFrag* acc) {
  (void)counters;
  (void)phase;
  const auto& p = *static_cast<const MokActResidue*>(static_cast<const pipelink_host_view*>(view)->residue);
  if (pipelink_mok_clamp())
    mok_act_owner::forward<true>(p, *task, *acc);
  else
    mok_act_owner::forward<false>(p, *task, *acc);
}
#else  // PIPELINK_EMIT: host-evaluated annotations only
#include "../include/mok_abi.h"
#endif

PL_STAGE("mok.act", "0.1.0-gptoss");
PL_PARAMS(MokActResidue);
PL_TOPOLOGY(true, "static");
// clamp on/off is a link-time variant (campaigns/mok/port/act_gptoss/act.cu:246-249)
PL_VARIANT(0, {{"pipelink_mok_clamp", 0}});
PL_VARIANT(1, {{"pipelink_mok_clamp", 1}});
PL_EXPORT(mok_act_init, mok_act_init, "extern \"C\" __device__ void mok_act_init(const void* view);");
PL_EXPORT(mok_act_fwd, mok_act_fwd,
          "extern \"C\" __device__ void mok_act_fwd(const void* view, const MokActTask* task, "
          "const MokCounters* counters, uint32_t* phase, const mok::AccFrag* acc);");
PL_SERVE(act_init, "mok_act_init");
PL_SERVE(act_fwd, "mok_act_fwd");
PL_USES("pipelink_mok_clamp");
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
