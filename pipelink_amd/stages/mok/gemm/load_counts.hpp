// The MoK GEMM owner's load accounting: how many of a wave's tile loads may still be in flight when it needs a given
// slot.  A wave's loads return in the order it issued them, so "the slot has landed" is "at most N loads are still
// outstanding" (s_waitcnt vmcnt(N)) with N = the loads issued after the slot's last one.  N too small only waits
// longer; N too large reads a buffer before its data is there.  Plain constexpr C++ on integers, so that a host
// compiler takes it too: the tests rebuild each wave's issue order load by load on the CPU and count.
#ifndef PIPELINK_MOK_GEMM_LOAD_COUNTS_HPP
#define PIPELINK_MOK_GEMM_LOAD_COUNTS_HPP

#ifndef MOK_COUNT_FN
#define MOK_COUNT_FN __device__ __forceinline__ constexpr
#endif

namespace mok_gemm_owner {
namespace counts {
constexpr int X_LOADS = 8;    // a wave's loads of one routed-row pair: 4 groups of 16 rows, two half-lines each
constexpr int W_LOADS = 4;    // a wave's loads of one weight slot: 4 groups of 16 rows
constexpr int FEW_DEPTH = 7;  // slots of the ring for tiles of few rows
constexpr int FEW_LOADS = W_LOADS + 1;  // a wave's tile loads of one of its slots

// tile loads issue_step(u) issues: routed rows, weight rows
template <int DEPTH>
MOK_COUNT_FN int x_loads_in(int u, int n) {
  const int s = u + DEPTH;
  const int pair = (u & 1) ? s - 1 : s;
  if (pair >= n) return 0;
  return DEPTH >= 4 ? X_LOADS / 2 : ((u & 1) == 0 ? X_LOADS : 0);
}
template <int DEPTH>
MOK_COUNT_FN int w_loads_in(int u, int n) { return u + DEPTH < n ? W_LOADS : 0; }
// Tile loads that may still be outstanding when slot `slot` is needed and steps up to `last`
// have been issued (step t waits for slot t+1 with last = t-1; the prologue waits for slot 0
// with last = -1).  The slot's weight rows are the last loads of step slot-DEPTH; its routed
// rows come no later, except that with split pairs groups 2-3 of an even slot are issued at
// the start of step slot+1-DEPTH.
template <int DEPTH>
MOK_COUNT_FN int loads_younger_than_slot(int slot, int last, int n) {
  int younger = 0;
  int first = slot + 1 - DEPTH;  // first step all of whose loads are younger
  if (DEPTH >= 4 && (slot & 1) == 0) {
    younger += w_loads_in<DEPTH>(first, n);
    ++first;
  }
  for (int u = first; u <= last; ++u) younger += x_loads_in<DEPTH>(u, n) + w_loads_in<DEPTH>(u, n);
  return younger;
}
// (ring for tiles of few rows) tile loads that may still be outstanding when slot `slot` is needed and steps up to
// `last` have been issued: step u issues all loads of slot u + FEW_DEPTH, the prologue (u < 0) those of the first
// FEW_DEPTH slots
MOK_COUNT_FN int few_younger(int slot, int last, int n) {
  int younger = 0;
  for (int u = slot + 1 - FEW_DEPTH; u <= last; ++u) younger += u + FEW_DEPTH < n ? FEW_LOADS : 0;
  return younger;
}

}  // namespace counts
}  // namespace mok_gemm_owner

#endif
