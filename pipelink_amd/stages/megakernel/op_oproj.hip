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
  for (int idx = threadIdx.x; idx < n; idx += MK_THREADS) {
    const int head = idx / MK_HEAD_DIM, d = idx % MK_HEAD_DIM;
    const float* p = m.attn_partial + (int64_t)head * m.chunks * (MK_HEAD_DIM + 2);
    float top = -1.0e30f;
    for (int c = 0; c < m.chunks; ++c) top = fmaxf(top, p[c * (MK_HEAD_DIM + 2) + MK_HEAD_DIM]);
    float o = 0.0f, l = 0.0f;
    for (int c = 0; c < m.chunks; ++c) {
      const float w = __builtin_amdgcn_exp2f(p[c * (MK_HEAD_DIM + 2) + MK_HEAD_DIM] - top);
      o += w * p[c * (MK_HEAD_DIM + 2) + d];
      l += w * p[c * (MK_HEAD_DIM + 2) + MK_HEAD_DIM + 1];
    }
    a[idx] = o / l;
  }
  __syncthreads();
  const uint16_t* w = mk::layer_of(m, instr->layer).wo;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int first, last;
  mk::my_rows(m.d, first, last);
  for (int r = first + wave; r < last; r += 4) {
    const float v = mk::row_dot(w + (int64_t)r * n, a, n, lane);
    if (lane == 0) m.x[r] += v;
  }
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
