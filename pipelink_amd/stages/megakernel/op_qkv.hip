// Package mk.qkv: qkv = Wqkv[layer] . vector; this workgroup's share of the (HQ + 2 HKV) * 64 rows.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_inputs_qkv(const void* view, MkPending* pending);

extern "C" __device__ void mk_qkv_op(const void* view, const MkInstr* instr, MkPending* pending) {
  const MkModel& m = mk::model(view);
  const uint16_t* w = mk::layer_of(m, instr->layer).wqkv;
  const float* x = mk::vec();
  int first, last;
  mk::my_rows((m.hq + 2 * m.hkv) * MK_HEAD_DIM, first, last);
  mk::matvec<3>(w, m.d, x, first, last, [&](int r, float v) { mk::shared_store(m.qkv + r, v); }, [&] { pipelink_call_inputs_qkv(view, pending); });
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.qkv", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_qkv, mk_qkv_op, "extern \"C\" __device__ void mk_qkv_op(const void* view, const MkInstr* instr, MkPending* pending);");
PL_CALL(inputs_qkv, "inputs_qkv", "extern \"C\" __device__ void pipelink_call_inputs_qkv(const void* view, MkPending* pending);");
PL_SERVE(op_qkv, "op_qkv");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_qkv", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
