// Package mk.rmsnorm: vector = x * rsqrt(mean(x^2) + eps) * weight into the workgroup's LDS vector.  Every
// workgroup normalises the whole residual for itself (D floats): cheaper than a grid barrier.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ int pipelink_mk_opcode_rmsnorm_ffn();
extern "C" __device__ int pipelink_mk_opcode_rmsnorm_final();

extern "C" __device__ void mk_rmsnorm_op(const void* view, const MkInstr* instr) {
  const MkModel& m = mk::model(view);
  const uint16_t* weight = instr->opcode == pipelink_mk_opcode_rmsnorm_final() ? mk::final_norm(m)
                           : instr->opcode == pipelink_mk_opcode_rmsnorm_ffn() ? mk::layer_of(m, instr->layer).ffn_norm
                                                                               : mk::layer_of(m, instr->layer).attn_norm;
  float* out = mk::vec();
  float* scratch = out + m.d;  // 4 floats behind the vector (the vector region holds at least D + 64 floats)
  const int tid = threadIdx.x;
  // a thread normalises the elements it loads (four at a time), and asks for their weights in the same breath: one
  // trip to memory, not two (the first 2048 elements' weights; longer vectors fetch the rest when they get there)
  constexpr int AHEAD = 2;
  uint2 wreg[AHEAD];
#pragma unroll
  for (int j = 0; j < AHEAD; ++j) {
    const int i = 4 * tid + 4 * MK_THREADS * j;
    wreg[j] = i < m.d ? *reinterpret_cast<const uint2*>(weight + i) : uint2{0u, 0u};
  }
  float ss = 0.0f;
  for (int i = 4 * tid; i < m.d; i += 4 * MK_THREADS) {  // D is a multiple of 512
    const mk::v4f v = mk::shared_load4(m.x, i, m.d);
    *reinterpret_cast<mk::v4f*>(out + i) = v;
    ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
  }
  ss = mk::wave_sum(ss);
  if ((tid & 63) == 0) scratch[tid >> 6] = ss;
  __syncthreads();
  const float inv = __builtin_amdgcn_rsqf((scratch[0] + scratch[1] + scratch[2] + scratch[3]) / (float)m.d + m.eps);
#pragma unroll
  for (int j = 0; j < AHEAD; ++j) {
    const int i = 4 * tid + 4 * MK_THREADS * j;
    if (i < m.d) {
      const mk::v4f v = *reinterpret_cast<const mk::v4f*>(out + i);  // this thread's own four
      *reinterpret_cast<mk::v4f*>(out + i) = mk::v4f{v.x * inv * mk::bf16_to_f32(wreg[j].x & 0xFFFFu), v.y * inv * __uint_as_float(wreg[j].x & 0xFFFF0000u),
                                                     v.z * inv * mk::bf16_to_f32(wreg[j].y & 0xFFFFu), v.w * inv * __uint_as_float(wreg[j].y & 0xFFFF0000u)};
    }
  }
  for (int i = 4 * tid + 4 * MK_THREADS * AHEAD; i < m.d; i += 4 * MK_THREADS) {
    const mk::v4f v = *reinterpret_cast<const mk::v4f*>(out + i);
    const uint2 w = *reinterpret_cast<const uint2*>(weight + i);
    *reinterpret_cast<mk::v4f*>(out + i) = mk::v4f{v.x * inv * mk::bf16_to_f32(w.x & 0xFFFFu), v.y * inv * __uint_as_float(w.x & 0xFFFF0000u),
                                                   v.z * inv * mk::bf16_to_f32(w.y & 0xFFFFu), v.w * inv * __uint_as_float(w.y & 0xFFFF0000u)};
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.rmsnorm", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_rmsnorm, mk_rmsnorm_op, "extern \"C\" __device__ void mk_rmsnorm_op(const void* view, const MkInstr* instr);");
PL_SERVE(op_rmsnorm, "op_rmsnorm");
PL_USES("pipelink_mk_vec");
PL_USES("pipelink_mk_opcode_rmsnorm_ffn");
PL_USES("pipelink_mk_opcode_rmsnorm_final");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_rmsnorm_attn", "opcode", 1, 1, "kernel");
PL_CLAIM("pipelink_mk_opcode_rmsnorm_ffn", "opcode", 1, 1, "kernel");
PL_CLAIM("pipelink_mk_opcode_rmsnorm_final", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
