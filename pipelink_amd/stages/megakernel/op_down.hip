// Package mk.down: x += Wdown[layer] . h for this workgroup's share of the D rows; h (DFF floats) is first
// copied into the workgroup's LDS vector.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_inputs_down(const void* view, MkPending* pending);

extern "C" __device__ void mk_down_op(const void* view, const MkInstr* instr, MkPending* pending) {
  const MkModel& m = mk::model(view);
  float* hv = mk::vec();
  float* scratch = hv + 8192;  // behind the vector
  const uint16_t* w = mk::layer_of(m, instr->layer).wdown;
  int first, last;
  mk::my_rows(m.d, first, last);
  // this workgroup's first eight rows of the matrix are asked for first (they depend on nobody); then, once the other
  // workgroups' intermediate is there, the intermediate and the residual the rows add to: all on their way at once
  mk::v4i wreg[8][4];
  if (first + 8 <= last) mk::split_load<8>(w + (int64_t)first * m.dff, m.dff, wreg);
  pipelink_call_inputs_down(view, pending);
  mk::v4f hreg[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) hreg[j] = mk::shared_load4(m.h, 4 * (int)threadIdx.x + 4 * MK_THREADS * j, m.dff);  // past DFF: zeros
  float xold = (int)threadIdx.x < 8 && first + (int)threadIdx.x < last ? mk::shared_load(m.x + first + threadIdx.x) : 0.0f;
#pragma unroll
  for (int j = 0; j < 8; ++j)
    if (4 * (int)threadIdx.x + 4 * MK_THREADS * j < m.dff) *reinterpret_cast<mk::v4f*>(hv + 4 * threadIdx.x + 4 * MK_THREADS * j) = hreg[j];
  __syncthreads();
  int r = first;
  for (; r + 8 <= last; r += 8) {
    if (r != first) {
      mk::split_load<8>(w + (int64_t)r * m.dff, m.dff, wreg);
      xold = (int)threadIdx.x < 8 ? mk::shared_load(m.x + r + threadIdx.x) : 0.0f;
    }
    mk::matvec_split<8>(w + (int64_t)r * m.dff, m.dff, hv, scratch, 8, wreg, [&](int i, float v) { mk::shared_store(m.x + r + i, xold + v); });
  }
  mk::matvec<1>(w, m.dff, hv, r, last, [&](int row, float v) { mk::shared_store(m.x + row, mk::shared_load(m.x + row) + v); });
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.down", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_down, mk_down_op, "extern \"C\" __device__ void mk_down_op(const void* view, const MkInstr* instr, MkPending* pending);");
PL_CALL(inputs_down, "inputs_down", "extern \"C\" __device__ void pipelink_call_inputs_down(const void* view, MkPending* pending);");
PL_SERVE(op_down, "op_down");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_down", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
