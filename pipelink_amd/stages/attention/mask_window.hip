// Package fa.mask.window: a query sees the `window` keys that end at its own position (causal sliding window; the
// reference's stage_mask_window.cu: kv_pos > q_pos - mask_param).  The window comes from this package's params.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include "include/fa_abi.h"

namespace fa_mask_window {
__device__ __forceinline__ int window(const void* view) {
  return static_cast<const FaMaskParams*>(static_cast<const pipelink_host_view*>(view)->residue)->window;
}
}  // namespace fa_mask_window

// number of leading keys any of the queries [q_first, q_last] may see (the core streams that many)
extern "C" __device__ int fa_mask_window_key_count(const void* view, int q_first, int q_last) {
  (void)view;
  (void)q_first;
  return q_last + 1;
}
// the first key any of the queries [q_first, q_last] may see (the core starts streaming at its block)
extern "C" __device__ int fa_mask_window_key_begin(const void* view, int q_first, int q_last) {
  (void)q_last;
  const int first = q_first - fa_mask_window::window(view) + 1;
  return first > 0 ? first : 0;
}
// 1 if every query of [q_first, q_last] sees every key of [k_first, k_last]: no per-element test needed
extern "C" __device__ int fa_mask_window_all_visible(const void* view, int q_first, int q_last, int k_first, int k_last) {
  return k_last <= q_first && k_first > q_last - fa_mask_window::window(view);
}
extern "C" __device__ int fa_mask_window_visible(const void* view, int q, int k) {
  return k <= q && k > q - fa_mask_window::window(view);
}
#else
#include "include/fa_abi.h"
#endif

PL_STAGE("fa.mask.window", "0.1.0");
PL_PARAMS(FaMaskParams);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_EXPORT(mask_key_count, fa_mask_window_key_count,
          "extern \"C\" __device__ int fa_mask_window_key_count(const void* view, int q_first, int q_last);");
PL_EXPORT(mask_key_begin, fa_mask_window_key_begin,
          "extern \"C\" __device__ int fa_mask_window_key_begin(const void* view, int q_first, int q_last);");
PL_EXPORT(mask_all_visible, fa_mask_window_all_visible,
          "extern \"C\" __device__ int fa_mask_window_all_visible(const void* view, int q_first, int q_last, int k_first, int k_last);");
PL_EXPORT(mask_visible, fa_mask_window_visible,
          "extern \"C\" __device__ int fa_mask_window_visible(const void* view, int q, int k);");
PL_SERVE(mask_key_count, "mask_key_count");
PL_SERVE(mask_key_begin, "mask_key_begin");
PL_SERVE(mask_all_visible, "mask_all_visible");
PL_SERVE(mask_visible, "mask_visible");
PL_PRELUDE("include/fa_abi.h");
PL_EMIT_MAIN()
