// Package mk.oproj: combines the attention chunks of every head into the workgroup's LDS vector (softmax over
// the whole context = the chunks' partial sums rescaled to a common maximum), then x += Wo[layer] . attention
// for this workgroup's share of the D rows.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_inputs_oproj(const void* view, MkPending* pending);

extern "C" __device__ void mk_oproj_op(const void* view, const MkInstr* instr, MkPending* pending) {
  const MkModel& m = mk::model(view);
  float* a = mk::vec();
  const int n = m.hq * MK_HEAD_DIM, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int pairs = m.hq * m.chunks, count = pairs * MK_PARTIAL_STRIDE;
  float* cmax = a + n;  // per (head, chunk), in LDS behind the vector: maximum, sum, then its weight in the whole softmax
  float* csum = cmax + pairs;
  float* weight = csum + pairs;
  const uint16_t* w = mk::layer_of(m, instr->layer).wo;
  int first, last;
  mk::my_rows(m.d, first, last);
  // Everything this op reads from memory is asked for before anything is used: the wave's first two matrix rows
  // (before the attention workgroups are waited for: the rows depend on nobody), then the chunks' maxima and sums,
  // the first eight chunks of the partial outputs (two items of four floats per thread) and the residual the
  // rows add to.
  constexpr int R = 2, CHUNKS_AHEAD = 8, ITEMS = 2;
  const int row0 = first + R * wave;
  mk::v4i wreg[R][4];
  const bool rows_ahead = row0 + R <= last;
  if (rows_ahead) mk::rows_load<R>(w + (int64_t)row0 * n, n, n, lane, wreg);
  pipelink_call_inputs_oproj(view, pending);
  mk::v4f stat = {0.0f, 0.0f, 0.0f, 0.0f};
  if (tid < pairs) stat = mk::shared_load4(m.attn_partial, tid * MK_PARTIAL_STRIDE + MK_HEAD_DIM, count);
  mk::v4f part[ITEMS][CHUNKS_AHEAD];
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int item = tid + MK_THREADS * it, head = item / (MK_HEAD_DIM / 4), d = 4 * (item % (MK_HEAD_DIM / 4));
#pragma unroll
    for (int c = 0; c < CHUNKS_AHEAD; ++c)  // an index past the buffer reads zeros
      part[it][c] = mk::shared_load4(m.attn_partial, item < n / 4 && c < m.chunks ? (head * m.chunks + c) * MK_PARTIAL_STRIDE + d : count, count);
  }
  float xold[R] = {};
  if (rows_ahead) {
#pragma unroll
    for (int i = 0; i < R; ++i) xold[i] = mk::shared_load(m.x + row0 + i);
  }
  if (tid < pairs) {
    cmax[tid] = stat.x;
    csum[tid] = stat.y;
  }
  for (int i = tid + MK_THREADS; i < pairs; i += MK_THREADS) {  // more than one workgroup's worth of pairs
    const mk::v4f t = mk::shared_load4(m.attn_partial, i * MK_PARTIAL_STRIDE + MK_HEAD_DIM, count);
    cmax[i] = t.x;
    csum[i] = t.y;
  }
  __syncthreads();
  for (int i = tid; i < pairs; i += MK_THREADS) {
    const int first_of_head = i / m.chunks * m.chunks;
    float top = -1.0e30f, l = 0.0f;
    for (int c = 0; c < m.chunks; ++c) top = fmaxf(top, cmax[first_of_head + c]);
    for (int c = 0; c < m.chunks; ++c) l += __builtin_amdgcn_exp2f(cmax[first_of_head + c] - top) * csum[first_of_head + c];
    weight[i] = __builtin_amdgcn_exp2f(cmax[i] - top) / l;
  }
  __syncthreads();
#pragma unroll
  for (int it = 0; it < ITEMS; ++it) {
    const int item = tid + MK_THREADS * it, head = item / (MK_HEAD_DIM / 4), d = 4 * (item % (MK_HEAD_DIM / 4));
    if (item >= n / 4) break;
    mk::v4f o = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int c = 0; c < CHUNKS_AHEAD; ++c) o += (c < m.chunks ? weight[head * m.chunks + c] : 0.0f) * part[it][c];
    for (int c = CHUNKS_AHEAD; c < m.chunks; ++c) o += weight[head * m.chunks + c] * mk::shared_load4(m.attn_partial, (head * m.chunks + c) * MK_PARTIAL_STRIDE + d, count);
    *reinterpret_cast<mk::v4f*>(a + 4 * item) = o;
  }
  for (int item = tid + MK_THREADS * ITEMS; item < n / 4; item += MK_THREADS) {  // more than 2048 attention outputs
    const int head = item / (MK_HEAD_DIM / 4), d = 4 * (item % (MK_HEAD_DIM / 4));
    mk::v4f o = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = 0; c < m.chunks; ++c) o += weight[head * m.chunks + c] * mk::shared_load4(m.attn_partial, (head * m.chunks + c) * MK_PARTIAL_STRIDE + d, count);
    *reinterpret_cast<mk::v4f*>(a + 4 * item) = o;
  }
  __syncthreads();
  if (rows_ahead) {
    float sum[R];
    mk::rows_dot<R>(w + (int64_t)row0 * n, n, a, n, lane, sum, &wreg);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < R; ++i) mk::shared_store(m.x + row0 + i, xold[i] + sum[i]);
    }
  }
  // the rest of this workgroup's rows (more than eight, or a group that is not whole)
  mk::matvec<R>(w, n, a, min(first + 4 * R, last), last, [&](int r, float v) { mk::shared_store(m.x + r, mk::shared_load(m.x + r) + v); });
  if (!rows_ahead && row0 < last) {  // fewer than R rows were left for this wave in the first eight
    for (int r = row0; r < min(row0 + R, last); ++r) {
      float sum[1];
      mk::rows_dot<1>(w + (int64_t)r * n, n, a, n, lane, sum);
      if (lane == 0) mk::shared_store(m.x + r, mk::shared_load(m.x + r) + sum[0]);
    }
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.oproj", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_oproj, mk_oproj_op, "extern \"C\" __device__ void mk_oproj_op(const void* view, const MkInstr* instr, MkPending* pending);");
PL_CALL(inputs_oproj, "inputs_oproj", "extern \"C\" __device__ void pipelink_call_inputs_oproj(const void* view, MkPending* pending);");
PL_SERVE(op_oproj, "op_oproj");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_oproj", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
