// Package mk.attn: decode attention of one (query head, chunk of the context) per workgroup -- scores of the
// head's rotated query against the chunk's keys, a local softmax, the unnormalised weighted sum of the values --
// and the append of the step's rotated key and value to the cache.  The output projection combines the chunks.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ float pipelink_call_rope_apply(const void* view, const float* v, int i);

namespace mk_attn {
__device__ __forceinline__ float bf16_round(float x) {
  uint32_t u = __float_as_uint(x);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  return __uint_as_float(u);
}
}  // namespace mk_attn

extern "C" __device__ void mk_attn_op(const void* view, const MkInstr* instr) {
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
  else if (tid < 128) knew[tid - 64] = mk_attn::bf16_round(pipelink_call_rope_apply(view, m.qkv + (m.hq + kvh) * MK_HEAD_DIM, tid - 64));
  __syncthreads();
  // ---- scores (log2 units) and the chunk's maximum ---------------------------------------------------------
  float local_max = -1.0e30f;
  for (int p = p0 + tid; p < p1; p += MK_THREADS) {
    float s = 0.0f;
    if (p < m.pos) {
      const mk::v4i* row = reinterpret_cast<const mk::v4i*>(kc + p * pos_stride);
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        const mk::v4i w = row[c];
        const uint32_t u[4] = {(uint32_t)w.x, (uint32_t)w.y, (uint32_t)w.z, (uint32_t)w.w};
#pragma unroll
        for (int e = 0; e < 4; ++e)
          s += mk::bf16_to_f32(u[e] & 0xFFFFu) * q[8 * c + 2 * e] + __uint_as_float(u[e] & 0xFFFF0000u) * q[8 * c + 2 * e + 1];
      }
    } else {
      for (int i = 0; i < 64; ++i) s += knew[i] * q[i];
    }
    s *= m.attn_scale_log2e;
    score[p - p0] = s;
    local_max = fmaxf(local_max, s);
  }
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
  // ---- unnormalised output: 16 lanes take one position (four d each, one 8-byte load), a wave four positions per
  // load instruction and sixteen such loads in flight ------------------------------------------------------
  {
    const int g = lane >> 4, dq = lane & 15;
    const int cached_end = min(p1, m.pos), last_cached = max(m.pos - 1, 0);
    float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int pb = p0 + 4 * wave + g; pb < cached_end; pb += 16 * 16) {
      uint2 v[16];
#pragma unroll
      for (int j = 0; j < 16; ++j) v[j] = *reinterpret_cast<const uint2*>(vc + min(pb + 16 * j, last_cached) * pos_stride + 4 * dq);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const int p = pb + 16 * j;
        const float s = p < cached_end ? score[p - p0] : 0.0f;
        o[0] += s * mk::bf16_to_f32(v[j].x & 0xFFFFu);
        o[1] += s * __uint_as_float(v[j].x & 0xFFFF0000u);
        o[2] += s * mk::bf16_to_f32(v[j].y & 0xFFFFu);
        o[3] += s * __uint_as_float(v[j].y & 0xFFFF0000u);
      }
    }
    if (p0 <= m.pos && m.pos < p1 && wave == 0 && g == 0) {  // the step's own token, as the cache will hold it
      const float s = score[m.pos - p0];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] += s * mk_attn::bf16_round(mk::shared_load(vnew + 4 * dq + e));
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      o[e] += __shfl_xor(o[e], 16);
      o[e] += __shfl_xor(o[e], 32);
    }
    if (g == 0) {
#pragma unroll
      for (int e = 0; e < 4; ++e) part[wave * 64 + 4 * dq + e] = o[e];
    }
  }
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
    vdst[tid] = (uint16_t)(__float_as_uint(mk_attn::bf16_round(mk::shared_load(vnew + tid))) >> 16);
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.attn", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_attn, mk_attn_op, "extern \"C\" __device__ void mk_attn_op(const void* view, const MkInstr* instr);");
PL_SERVE(op_attn, "op_attn");
PL_CALL(rope_apply, "rope_apply", "extern \"C\" __device__ float pipelink_call_rope_apply(const void* view, const float* v, int i);");
PL_USES("pipelink_mk_vec");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
