// Package mk.lmhead: logits = Wlm . vector for this workgroup's share of the vocabulary rows.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_inputs_lmhead(const void* view, MkPending* pending);

extern "C" __device__ void mk_lmhead_op(const void* view, const MkInstr* instr, MkPending* pending) {
  (void)instr;
  const MkModel& m = mk::model(view);
  const uint16_t* w = mk::lm_head(m);
  const float* x = mk::vec();
  int first, last;
  mk::my_rows(m.vocab, first, last);
  mk::matvec<4>(w, m.d, x, first, last, [&](int r, float v) { m.logits[r] = v; }, [&] { pipelink_call_inputs_lmhead(view, pending); });
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.lmhead", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(op_lmhead, mk_lmhead_op, "extern \"C\" __device__ void mk_lmhead_op(const void* view, const MkInstr* instr, MkPending* pending);");
PL_CALL(inputs_lmhead, "inputs_lmhead", "extern \"C\" __device__ void pipelink_call_inputs_lmhead(const void* view, MkPending* pending);");
PL_SERVE(op_lmhead, "op_lmhead");
PL_USES("pipelink_mk_vec");
// the number(s) the instruction stream calls this op by: one slot each in the link's opcode domain
PL_CLAIM("pipelink_mk_opcode_lmhead", "opcode", 1, 1, "kernel");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
