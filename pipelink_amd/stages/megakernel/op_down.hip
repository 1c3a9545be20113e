// Package mk.down: x += Wdown[layer] . h for this workgroup's share of the D rows; h (DFF floats) is first
// copied into the workgroup's LDS vector.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void mk_down_op(const void* view, const MkInstr* instr) {
  const MkModel& m = mk::model(view);
  float* hv = mk::vec();
  for (int i = threadIdx.x; i < m.dff; i += MK_THREADS) hv[i] = m.h[i];
  __syncthreads();
  const uint16_t* w = mk::layer_of(m, instr->layer).wdown;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int first, last;
  mk::my_rows(m.d, first, last);
  for (int r = first + wave; r < last; r += 4) {
    const float v = mk::row_dot(w + (int64_t)r * m.dff, hv, m.dff, lane);
    if (lane == 0) m.x[r] += v;
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.down", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_down, mk_down_op, "extern \"C\" __device__ void mk_down_op(const void* view, const MkInstr* instr);");
PL_SERVE(op_down, "op_down");
PL_USES("pipelink_mk_vec");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
