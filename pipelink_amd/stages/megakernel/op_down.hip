// Package mk.down: x += Wdown[layer] . h for this workgroup's share of the D rows; h (DFF floats) is first
// copied into the workgroup's LDS vector.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void mk_down_op(const void* view, const MkInstr* instr) {
  const MkModel& m = mk::model(view);
  float* hv = mk::vec();
  for (int i = 4 * threadIdx.x; i < m.dff; i += 4 * MK_THREADS) *reinterpret_cast<mk::v4f*>(hv + i) = mk::shared_load4(m.h, i, m.dff);
  __syncthreads();
  const uint16_t* w = mk::layer_of(m, instr->layer).wdown;
  float* scratch = hv + 8192;  // behind the vector
  int first, last;
  mk::my_rows(m.d, first, last);
  for (int r = first; r < last; r += 8) {
    const int count = min(8, last - r);
    if (count == 8) {
      mk::matvec_split<8>(w + (int64_t)r * m.dff, m.dff, hv, scratch, 8, [&](int i, float v) { mk::shared_store(m.x + r + i, mk::shared_load(m.x + r + i) + v); });
    } else {
      mk::matvec<1>(w, m.dff, hv, r, last, [&](int row, float v) { mk::shared_store(m.x + row, mk::shared_load(m.x + row) + v); });
    }
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
