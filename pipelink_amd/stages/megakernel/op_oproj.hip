// Package mk.oproj: combines the attention chunks of every head into the workgroup's LDS vector (softmax over
// the whole context = the chunks' partial sums rescaled to a common maximum), then x += Wo[layer] . attention
// for this workgroup's share of the D rows.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void mk_oproj_op(const void* view, const MkInstr* instr) {
  const MkModel& m = mk::model(view);
  float* a = mk::vec();
  const int n = m.hq * MK_HEAD_DIM;
  // per (head, chunk): its weight exp2(max_c - max) / sum in the softmax over the whole context, into LDS behind the vector
  const int pairs = m.hq * m.chunks, count = pairs * MK_PARTIAL_STRIDE;
  float* cmax = a + n;
  float* csum = cmax + pairs;
  float* weight = csum + pairs;
  for (int i = threadIdx.x; i < pairs; i += MK_THREADS) {
    const mk::v4f t = mk::shared_load4(m.attn_partial, i * MK_PARTIAL_STRIDE + MK_HEAD_DIM, count);
    cmax[i] = t.x;
    csum[i] = t.y;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < pairs; i += MK_THREADS) {
    const int first_of_head = i / m.chunks * m.chunks;
    float top = -1.0e30f, l = 0.0f;
    for (int c = 0; c < m.chunks; ++c) top = fmaxf(top, cmax[first_of_head + c]);
    for (int c = 0; c < m.chunks; ++c) l += __builtin_amdgcn_exp2f(cmax[first_of_head + c] - top) * csum[first_of_head + c];
    weight[i] = __builtin_amdgcn_exp2f(cmax[i] - top) / l;
  }
  __syncthreads();
  for (int item = threadIdx.x; item < n / 4; item += MK_THREADS) {  // four outputs of one head per thread
    const int head = item / (MK_HEAD_DIM / 4), d = 4 * (item % (MK_HEAD_DIM / 4));
    mk::v4f o = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int c = 0; c < m.chunks; c += 4) {  // four chunks' loads in flight; a chunk past the last reads past the buffer: zeros
      mk::v4f part[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) part[j] = mk::shared_load4(m.attn_partial, c + j < m.chunks ? (head * m.chunks + c + j) * MK_PARTIAL_STRIDE + d : count, count);
#pragma unroll
      for (int j = 0; j < 4; ++j) o += (c + j < m.chunks ? weight[head * m.chunks + c + j] : 0.0f) * part[j];
    }
    *reinterpret_cast<mk::v4f*>(a + 4 * item) = o;
  }
  __syncthreads();
  const uint16_t* w = mk::layer_of(m, instr->layer).wo;
  int first, last;
  mk::my_rows(m.d, first, last);
  mk::matvec<2>(w, n, a, first, last, [&](int r, float v) { mk::shared_store(m.x + r, mk::shared_load(m.x + r) + v); });
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.oproj", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_oproj, mk_oproj_op, "extern \"C\" __device__ void mk_oproj_op(const void* view, const MkInstr* instr);");
PL_SERVE(op_oproj, "op_oproj");
PL_USES("pipelink_mk_vec");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
