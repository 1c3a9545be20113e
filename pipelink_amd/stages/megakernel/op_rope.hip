// Package mk.rope: rotary embedding of one 64-element head vector at the step's position (rotate-half
// pairing: element i with i + 32; cos / sin come in a table the host fills for the position).
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

// out[i] for lane-held element i of head vector `v` (64 floats of the qkv buffer)
extern "C" __device__ float mk_rope_apply(const void* view, const float* v, int i) {
  const MkModel& m = mk::model(view);
  const int j = i & 31;
  const float c = m.rope[j], s = m.rope[32 + j];
  const float a = mk::shared_load(v + i), b = mk::shared_load(v + (i < 32 ? i + 32 : i - 32));
  return i < 32 ? a * c - b * s : a * c + b * s;
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.rope", "0.1.0");
PL_NO_PARAMS();
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_EXPORT(rope_apply, mk_rope_apply, "extern \"C\" __device__ float mk_rope_apply(const void* view, const float* v, int i);");
PL_SERVE(rope_apply, "rope_apply");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
