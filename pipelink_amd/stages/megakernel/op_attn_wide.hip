// Package mk.attn.wide: decode attention of one (query head, chunk of the context) per workgroup -- scores of the
// head's rotated query against the chunk's keys, a local softmax, the unnormalised weighted sum of the values --
// and the append of the step's rotated key and value to the cache.  The output projection combines the chunks.
// Same contract as mk.attn; the scores are computed the other way round: a wave takes a position and its 64
// lanes the 64 elements of the dot product (coalesced 128-byte key rows), where mk.attn gives each thread a
// position of its own.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ float pipelink_call_rope_apply(const void* view, const float* v, int i);

namespace mk_attn_wide {
__device__ __forceinline__ float bf16_round(float x) {
  uint32_t u = __float_as_uint(x);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  return __uint_as_float(u);
}
}  // namespace mk_attn_wide

extern "C" __device__ void mk_attn_wide_op(const void* view, const MkInstr* instr) {
  const MkModel& m = mk::model(view);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int head = blockIdx.x / m.chunks, chunk = blockIdx.x % m.chunks;
  if (head >= m.hq) return;
  const int kvh = head / (m.hq / m.hkv);
  const int npos = m.pos + 1;  // the cache holds positions 0 .. pos - 1, the step's own token is position pos
  const int per = (npos + m.chunks - 1) / m.chunks;
  const int p0 = min(chunk * per, npos), p1 = min(p0 + per, npos);
  float* q = mk::vec();            // [64] rotated query
  float* knew = q + 64;            // [64] the step's rotated key, rounded to bf16 as the cache will hold it
  float* red = q + 128;            // [8] reduction scratch
  float* part = q + 256;           // [4][64] per-wave partial outputs
  float* score = q + 512;          // [per]
  const uint16_t* kc = m.kv_cache + (((int64_t)instr->layer * 2 + 0) * m.smax * m.hkv + kvh) * MK_HEAD_DIM;
  const uint16_t* vc = m.kv_cache + (((int64_t)instr->layer * 2 + 1) * m.smax * m.hkv + kvh) * MK_HEAD_DIM;
  const int64_t pos_stride = (int64_t)m.hkv * MK_HEAD_DIM;
  const float* vnew = m.qkv + (m.hq + m.hkv + kvh) * MK_HEAD_DIM;
  if (tid < 64) q[tid] = pipelink_call_rope_apply(view, m.qkv + head * MK_HEAD_DIM, tid);
  else if (tid < 128) knew[tid - 64] = mk_attn_wide::bf16_round(pipelink_call_rope_apply(view, m.qkv + (m.hq + kvh) * MK_HEAD_DIM, tid - 64));
  __syncthreads();
  // ---- scores (log2 units) and the chunk's maximum ---------------------------------------------------------
  float local_max = -1.0e30f;
  {
    const float ql = q[lane];
    int p = p0 + wave;
    for (; p + 28 < p1 && p + 28 < m.pos; p += 32) {
      float kv[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) kv[j] = mk::bf16_to_f32(kc[(p + 4 * j) * pos_stride + lane]) * ql;
#pragma unroll
      for (int sh = 32; sh >= 1; sh >>= 1)
#pragma unroll
        for (int j = 0; j < 8; ++j) kv[j] += __shfl_xor(kv[j], sh);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float sc = kv[j] * m.attn_scale_log2e;
        if (lane == 0) score[p + 4 * j - p0] = sc;
        local_max = fmaxf(local_max, sc);
      }
    }
    for (; p < p1; p += 4) {
      const float kv = p < m.pos ? mk::bf16_to_f32(kc[p * pos_stride + lane]) : knew[lane];
      const float sc = mk::wave_sum(kv * ql) * m.attn_scale_log2e;
      if (lane == 0) score[p - p0] = sc;
      local_max = fmaxf(local_max, sc);
    }
  }
  __syncthreads();
#pragma unroll
  for (int sh = 32; sh >= 1; sh >>= 1) local_max = fmaxf(local_max, __shfl_xor(local_max, sh));
  if (lane == 0) red[wave] = local_max;
  __syncthreads();
  const float cmax = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float local_sum = 0.0f;
  for (int p = p0 + tid; p < p1; p += MK_THREADS) {
    const float e = __builtin_amdgcn_exp2f(score[p - p0] - cmax);
    score[p - p0] = e;
    local_sum += e;
  }
  local_sum = mk::wave_sum(local_sum);
  if (lane == 0) red[4 + wave] = local_sum;
  __syncthreads();
  // ---- unnormalised output: lane = d, a wave takes every fourth position ------------------------------------
  float o = 0.0f;
  {
    int p = p0 + wave;
    for (; p + 28 < p1 && p + 28 < m.pos; p += 32) {  // eight cached positions at a time: eight loads in flight
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = mk::bf16_to_f32(vc[(p + 4 * j) * pos_stride + lane]);
#pragma unroll
      for (int j = 0; j < 8; ++j) o += score[p + 4 * j - p0] * v[j];
    }
    for (; p < p1; p += 4) {
      const float v = p < m.pos ? mk::bf16_to_f32(vc[p * pos_stride + lane]) : mk_attn_wide::bf16_round(mk::shared_load(vnew + lane));
      o += score[p - p0] * v;
    }
  }
  part[wave * 64 + lane] = o;
  __syncthreads();
  float* out = m.attn_partial + ((int64_t)head * m.chunks + chunk) * MK_PARTIAL_STRIDE;
  if (tid < 64) mk::shared_store(out + tid, part[tid] + part[64 + tid] + part[128 + tid] + part[192 + tid]);
  if (tid == 64) {
    mk::shared_store(out + MK_HEAD_DIM, cmax);
    mk::shared_store(out + MK_HEAD_DIM + 1, red[4] + red[5] + red[6] + red[7]);
  }
  // ---- append the step's key and value (one workgroup per KV head does it) ----------------------------------
  if (head % (m.hq / m.hkv) == 0 && p0 <= m.pos && m.pos < p1 && tid < 64) {
    uint16_t* kdst = m.kv_cache + (((int64_t)instr->layer * 2 + 0) * m.smax + m.pos) * pos_stride + kvh * MK_HEAD_DIM;
    uint16_t* vdst = m.kv_cache + (((int64_t)instr->layer * 2 + 1) * m.smax + m.pos) * pos_stride + kvh * MK_HEAD_DIM;
    kdst[tid] = (uint16_t)(__float_as_uint(knew[tid]) >> 16);
    vdst[tid] = (uint16_t)(__float_as_uint(mk_attn_wide::bf16_round(mk::shared_load(vnew + tid))) >> 16);
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.attn.wide", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_attn, mk_attn_wide_op, "extern \"C\" __device__ void mk_attn_wide_op(const void* view, const MkInstr* instr);");
PL_SERVE(op_attn, "op_attn");
PL_CALL(rope_apply, "rope_apply", "extern \"C\" __device__ float pipelink_call_rope_apply(const void* view, const float* v, int i);");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_attn", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
