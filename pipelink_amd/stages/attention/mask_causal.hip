// Package fa.mask.causal: a query sees the keys at or before its own position.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/fa_abi.h"

// number of leading keys any of the queries [q_first, q_last] may see (the core streams that many)
extern "C" __device__ int fa_mask_causal_key_count(const void* view, int q_first, int q_last) {
  (void)view;
  (void)q_first;
  return q_last + 1;
}
// the first key any of the queries [q_first, q_last] may see (the core starts streaming at its block)
extern "C" __device__ int fa_mask_causal_key_begin(const void* view, int q_first, int q_last) {
  (void)view;
  (void)q_first;
  (void)q_last;
  return 0;
}
// 1 if every query of [q_first, q_last] sees every key of [k_first, k_last]: no per-element test needed
extern "C" __device__ int fa_mask_causal_all_visible(const void* view, int q_first, int q_last, int k_first, int k_last) {
  (void)view;
  (void)q_last;
  (void)k_first;
  return k_last <= q_first;
}
extern "C" __device__ int fa_mask_causal_visible(const void* view, int q, int k) {
  (void)view;
  return k <= q;
}
#else
#include "include/fa_abi.h"
#endif

PL_STAGE("fa.mask.causal", "0.1.0");
PL_PARAMS(FaMaskParams);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_EXPORT(mask_key_count, fa_mask_causal_key_count,
          "extern \"C\" __device__ int fa_mask_causal_key_count(const void* view, int q_first, int q_last);");
PL_EXPORT(mask_key_begin, fa_mask_causal_key_begin,
          "extern \"C\" __device__ int fa_mask_causal_key_begin(const void* view, int q_first, int q_last);");
PL_EXPORT(mask_all_visible, fa_mask_causal_all_visible,
          "extern \"C\" __device__ int fa_mask_causal_all_visible(const void* view, int q_first, int q_last, int k_first, int k_last);");
PL_EXPORT(mask_visible, fa_mask_causal_visible,
          "extern \"C\" __device__ int fa_mask_causal_visible(const void* view, int q, int k);");
PL_SERVE(mask_key_count, "mask_key_count");
PL_SERVE(mask_key_begin, "mask_key_begin");
PL_SERVE(mask_all_visible, "mask_all_visible");
PL_SERVE(mask_visible, "mask_visible");
PL_PRELUDE("include/fa_abi.h");
PL_EMIT_MAIN()
