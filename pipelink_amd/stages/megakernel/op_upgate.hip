// Package mk.upgate: h = silu(Wgate . vector) * (Wup . vector) for this workgroup's share of the DFF rows.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_inputs_upgate(const void* view, MkPending* pending);

extern "C" __device__ void mk_upgate_op(const void* view, const MkInstr* instr, MkPending* pending) {
  const MkModel& m = mk::model(view);
  const mk::Layer l = mk::layer_of(m, instr->layer);
  const float* x = mk::vec();
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int first, last;
  mk::my_rows(m.dff, first, last);
  constexpr int R = 4;
  // Two sets of row registers, gate and up, each refilled with the wave's next four rows as soon as it has been used:
  // one set is always on its way.  The first gate rows are asked for before the vector they multiply is waited for.
  mk::v4i wg[R][4], wu[R][4];
  const int r0 = first + R * wave;
  if (r0 < last) mk::rows_load<R>(l.wgate + (int64_t)r0 * m.d, m.d, m.d, lane, wg);
  pipelink_call_inputs_upgate(view, pending);
  if (r0 < last) mk::rows_load<R>(l.wup + (int64_t)r0 * m.d, m.d, m.d, lane, wu);
  for (int r = r0; r < last; r += 4 * R) {  // DFF / workgroups is a multiple of 4 (the host checks)
    const int next = r + 4 * R;
    float g[R], u[R];
    mk::rows_dot<R>(l.wgate + (int64_t)r * m.d, m.d, x, m.d, lane, g, &wg);
    if (next < last) mk::rows_load<R>(l.wgate + (int64_t)next * m.d, m.d, m.d, lane, wg);
    mk::rows_dot<R>(l.wup + (int64_t)r * m.d, m.d, x, m.d, lane, u, &wu);
    if (next < last) mk::rows_load<R>(l.wup + (int64_t)next * m.d, m.d, m.d, lane, wu);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < R; ++i)
        if (r + i < last) mk::shared_store(m.h + r + i, g[i] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-g[i] * 1.4426950408889634f)) * u[i]);
    }
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.upgate", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_upgate, mk_upgate_op, "extern \"C\" __device__ void mk_upgate_op(const void* view, const MkInstr* instr, MkPending* pending);");
PL_CALL(inputs_upgate, "inputs_upgate", "extern \"C\" __device__ void pipelink_call_inputs_upgate(const void* view, MkPending* pending);");
PL_SERVE(op_upgate, "op_upgate");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_upgate", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
