// Package mk.attn.wide: decode attention of one (query head, chunk of the context) per workgroup -- scores of the
// head's rotated query against the chunk's keys, a local softmax, the unnormalised weighted sum of the values --
// and the append of the step's rotated key and value to the cache.  The output projection combines the chunks.
// Same contract as mk.attn with the work cut the other way: sixteen lanes take one cached position (four elements
// each, 8-byte loads) where mk.attn gives it eight lanes and 16-byte loads -- twice the load instructions in
// flight per wave, and the value pass needs no exchange between lanes (a row of 16 lanes owns a position).
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ float pipelink_call_rope_apply(const void* view, const float* v, int i);
extern "C" __device__ void pipelink_call_inputs_attn(const void* view, MkPending* pending);

namespace mk_attn_wide {
__device__ __forceinline__ float bf16_round(float x) {
  uint32_t u = __float_as_uint(x);
  u = (u + 0x7FFFu + ((u >> 16) & 1u)) & 0xFFFF0000u;
  return __uint_as_float(u);
}
}  // namespace mk_attn_wide

extern "C" __device__ void mk_attn_wide_op(const void* view, const MkInstr* instr, MkPending* pending) {
  const MkModel& m = mk::model(view);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int head = blockIdx.x / m.chunks, chunk = blockIdx.x % m.chunks;
  if (head >= m.hq) return;
  const int kvh = head / (m.hq / m.hkv);
  const int npos = m.pos + 1;  // the cache holds positions 0 .. pos - 1, the step's own token is position pos
  // the cached positions are dealt evenly to the chunks; the last chunk takes the step's own token as well
  const int per = (m.pos + m.chunks - 1) / m.chunks;
  const int p0 = min(chunk * per, m.pos), p1 = chunk == m.chunks - 1 ? npos : min(p0 + per, m.pos);
  float* q = mk::vec();            // [64] rotated query
  float* knew = q + 64;            // [64] the step's rotated key, rounded to bf16 as the cache will hold it
  float* red = q + 128;            // [8] reduction scratch
  float* part = q + 256;           // [16][64] partial outputs, one per row of 16 lanes
  float* score = q + 1280;         // [per + 1]
  const uint16_t* kc = m.kv_cache + (((int64_t)instr->layer * 2 + 0) * m.smax * m.hkv + kvh) * MK_HEAD_DIM;
  const uint16_t* vc = m.kv_cache + (((int64_t)instr->layer * 2 + 1) * m.smax * m.hkv + kvh) * MK_HEAD_DIM;
  const int64_t pos_stride = (int64_t)m.hkv * MK_HEAD_DIM;
  const float* vnew = m.qkv + (m.hq + m.hkv + kvh) * MK_HEAD_DIM;
  // Sixteen lanes take one position (four elements each, one 8-byte load), a wave four positions per load
  // instruction, the workgroup 16.  The first 32 such loads of the keys and of the values (512 positions) are
  // asked for before the query is rotated: neither depends on it.
  constexpr int AHEAD = 32;
  const int cached_end = min(p1, m.pos), last_cached = max(m.pos - 1, 0);
  const int g = lane >> 4, piece = lane & 15, pl0 = p0 + 4 * wave + g;
  uint2 kreg[AHEAD], vreg[AHEAD];
#pragma unroll
  for (int j = 0; j < AHEAD; ++j) kreg[j] = *reinterpret_cast<const uint2*>(kc + min(pl0 + 16 * j, last_cached) * pos_stride + 4 * piece);
#pragma unroll
  for (int j = 0; j < AHEAD; ++j) vreg[j] = *reinterpret_cast<const uint2*>(vc + min(pl0 + 16 * j, last_cached) * pos_stride + 4 * piece);
  pipelink_call_inputs_attn(view, pending);  // the cache reads above depend on nobody; the query, key and value of this step do
  if (tid < 64) q[tid] = pipelink_call_rope_apply(view, m.qkv + head * MK_HEAD_DIM, tid);
  else if (tid < 128) knew[tid - 64] = mk_attn_wide::bf16_round(pipelink_call_rope_apply(view, m.qkv + (m.hq + kvh) * MK_HEAD_DIM, tid - 64));
  __syncthreads();
  // ---- scores (log2 units) and the chunk's maximum ---------------------------------------------------------
  float local_max = -1.0e30f;
  {
    const mk::v4f q4 = *reinterpret_cast<const mk::v4f*>(q + 4 * piece);
    for (int pb = pl0; pb < cached_end; pb += 16 * AHEAD) {
      if (pb != pl0) {
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) kreg[j] = *reinterpret_cast<const uint2*>(kc + min(pb + 16 * j, last_cached) * pos_stride + 4 * piece);
      }
#pragma unroll
      for (int j = 0; j < AHEAD; ++j) {
        float part4 = mk::bf16_to_f32(kreg[j].x & 0xFFFFu) * q4.x + __uint_as_float(kreg[j].x & 0xFFFF0000u) * q4.y +
                      mk::bf16_to_f32(kreg[j].y & 0xFFFFu) * q4.z + __uint_as_float(kreg[j].y & 0xFFFF0000u) * q4.w;
        part4 = mk::sum8_first(part4);            // lanes 0 and 8 of the row: the sums of its two halves
        part4 += mk::dpp<0x108>(part4);           // lane 0: + the lane eight further on
        const float sc = part4 * m.attn_scale_log2e;
        const int p = pb + 16 * j;
        if (p < cached_end && piece == 0) {
          score[p - p0] = sc;
          local_max = fmaxf(local_max, sc);
        }
      }
    }
    if (p0 <= m.pos && m.pos < p1 && wave == 0) {  // the step's own token
      const float sc = mk::wave_sum(knew[lane] * q[lane]) * m.attn_scale_log2e;
      if (lane == 0) score[m.pos - p0] = sc;
      local_max = fmaxf(local_max, sc);
    }
  }
  local_max = mk::wave_max(local_max);
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
  // ---- unnormalised output -----------------------------------------------------------------------------------
  {
    float o[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int pb = pl0; pb < cached_end; pb += 16 * AHEAD) {
      if (pb != pl0) {
#pragma unroll
        for (int j = 0; j < AHEAD; ++j) vreg[j] = *reinterpret_cast<const uint2*>(vc + min(pb + 16 * j, last_cached) * pos_stride + 4 * piece);
      }
#pragma unroll
      for (int j = 0; j < AHEAD; ++j) {
        const int p = pb + 16 * j;
        const float sc = p < cached_end ? score[p - p0] : 0.0f;
        o[0] += sc * mk::bf16_to_f32(vreg[j].x & 0xFFFFu);
        o[1] += sc * __uint_as_float(vreg[j].x & 0xFFFF0000u);
        o[2] += sc * mk::bf16_to_f32(vreg[j].y & 0xFFFFu);
        o[3] += sc * __uint_as_float(vreg[j].y & 0xFFFF0000u);
      }
    }
    if (p0 <= m.pos && m.pos < p1 && wave == 0 && g == 0) {  // the step's own token, as the cache will hold it
      const float sc = score[m.pos - p0];
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] += sc * mk_attn_wide::bf16_round(mk::shared_load(vnew + 4 * piece + e));
    }
    // a row of 16 lanes holds one partial output: 16 rows per workgroup
    *reinterpret_cast<mk::v4f*>(part + (4 * wave + g) * 64 + 4 * piece) = mk::v4f{o[0], o[1], o[2], o[3]};
  }
  __syncthreads();
  float* out = m.attn_partial + ((int64_t)head * m.chunks + chunk) * MK_PARTIAL_STRIDE;
  if (tid < 64) {
    float sum = 0.0f;
#pragma unroll
    for (int row = 0; row < 16; ++row) sum += part[64 * row + tid];
    mk::shared_store(out + tid, sum);
  }
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
PL_EXPORT(op_attn, mk_attn_wide_op, "extern \"C\" __device__ void mk_attn_wide_op(const void* view, const MkInstr* instr, MkPending* pending);");
PL_CALL(inputs_attn, "inputs_attn", "extern \"C\" __device__ void pipelink_call_inputs_attn(const void* view, MkPending* pending);");
PL_SERVE(op_attn, "op_attn");
PL_CALL(rope_apply, "rope_apply", "extern \"C\" __device__ float pipelink_call_rope_apply(const void* view, const float* v, int i);");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_attn", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
