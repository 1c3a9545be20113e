"""The MoK GEMM owner's wait counts, checked against a wave's issue order rebuilt load by load on the CPU.

``pipelink_amd/stages/mok/gemm/load_counts.hpp`` is the code the kernel compiles (every ``s_waitcnt vmcnt(N)`` of the
mainloops takes its N from it); g++ compiles it here with the device markers defined away.  The harness writes down,
for a contraction of n slots, every tile load a wave issues in the order the loader issues them -- schedule step by
schedule step, routed rows in front of weight rows, each load tagged with the slots whose buffers it fills -- and counts
the loads behind the last one a slot needs.  The formula must give exactly that number for every n, every step and both
ring depths: one more and a step reads a buffer before its data has landed, one fewer and it waits for a load it does
not need.
"""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GEMM = os.path.join(ROOT, "pipelink_amd", "stages", "mok", "gemm")

HARNESS = r"""
#define MOK_COUNT_FN constexpr inline
#include "load_counts.hpp"
#include <cstdio>
#include <vector>
using namespace mok_gemm_owner::counts;

struct Load { int step; int serves_lo, serves_hi; };  // fills the buffers of slots serves_lo .. serves_hi

// Full ring of depth DEPTH: schedule step u (u = -DEPTH .. n - 1; the negative ones are the prologue) first issues
// routed rows -- a pair of slots at a time, each load one half-line for the pair's first slot and one for its second:
// with DEPTH >= 4 half of the pair's loads on the even step, the other half on the odd step behind it, with DEPTH 2
// all of them on the even step -- then the weight rows of slot u + DEPTH.
template <int DEPTH>
static std::vector<Load> issue_order(int n, int last) {
  std::vector<Load> v;
  for (int u = -DEPTH; u <= last; ++u) {
    const int s = u + DEPTH;
    const int pair = (u & 1) ? s - 1 : s;
    if (pair < n) {
      const int loads = DEPTH >= 4 ? X_LOADS / 2 : ((u & 1) == 0 ? X_LOADS : 0);
      for (int i = 0; i < loads; ++i) v.push_back({u, pair, pair + 1});
    }
    if (s < n)
      for (int i = 0; i < W_LOADS; ++i) v.push_back({u, s, s});
  }
  return v;
}
// Ring for tiles of few rows: step u issues every load of slot u + FEW_DEPTH.
static std::vector<Load> issue_order_few(int n, int last) {
  std::vector<Load> v;
  for (int u = -FEW_DEPTH; u <= last; ++u)
    if (u + FEW_DEPTH < n)
      for (int i = 0; i < FEW_LOADS; ++i) v.push_back({u, u + FEW_DEPTH, u + FEW_DEPTH});
  return v;
}
static int behind_last_of(const std::vector<Load>& v, int slot) {
  int last_needed = -1;
  for (int i = 0; i < (int)v.size(); ++i)
    if (v[i].serves_lo <= slot && slot <= v[i].serves_hi) last_needed = i;
  return last_needed < 0 ? -1 : (int)v.size() - 1 - last_needed;
}
template <int DEPTH>
static int check(const char* name) {
  int bad = 0, checked = 0;
  for (int n = 1; n <= 64; ++n) {
    // the prologue waits for slot 0 with every negative step issued; step t waits for slot t + 1 with steps up to t - 1 issued
    for (int t = -1; t + 1 < n; ++t) {
      const int slot = t + 1, last = t - 1 < -1 ? -1 : t - 1;
      const int truth = behind_last_of(issue_order<DEPTH>(n, last), slot);
      const int formula = loads_younger_than_slot<DEPTH>(slot, last, n);
      ++checked;
      if (truth < 0 || formula != truth) {
        if (bad++ < 10) printf("%s: n %d slot %d last %d: formula %d, issue order %d\n", name, n, slot, last, formula, truth);
      }
    }
  }
  printf("%s: %d waits checked, %d wrong\n", name, checked, bad);
  return bad;
}
static int check_few() {
  int bad = 0, checked = 0;
  for (int n = 1; n <= 64; ++n)
    for (int t = -1; t + 1 < n; ++t) {
      const int slot = t + 1, last = t - 1 < -1 ? -1 : t - 1;
      const int truth = behind_last_of(issue_order_few(n, last), slot);
      const int formula = few_younger(slot, last, n);
      ++checked;
      if (truth < 0 || formula != truth || formula % FEW_LOADS != 0 || formula > (FEW_DEPTH - 1) * FEW_LOADS) {
        if (bad++ < 10) printf("few rows: n %d slot %d last %d: formula %d, issue order %d\n", n, slot, last, formula, truth);
      }
    }
  printf("few rows: %d waits checked, %d wrong\n", checked, bad);
  return bad;
}
// the compile-time uses: the steady state of the placed loop and the prologue of a long contraction
static_assert(loads_younger_than_slot<4>(101, 99, 1 << 20) == 2 * (W_LOADS + X_LOADS / 2), "even step, depth 4");
static_assert(loads_younger_than_slot<4>(102, 100, 1 << 20) == 2 * (W_LOADS + X_LOADS / 2) - X_LOADS / 2, "odd step, depth 4");
int main() {
  int bad = check<4>("depth 4") + check<2>("depth 2") + check_few();
  // the constant the prologue uses when the contraction has at least DEPTH slots is the run-time count for every such n
  for (int n = 4; n <= 64; ++n)
    if (loads_younger_than_slot<4>(0, -1, n) != loads_younger_than_slot<4>(0, -1, 1 << 20)) { printf("prologue constant differs at n %d\n", n); ++bad; }
  for (int n = 2; n <= 64; ++n)
    if (loads_younger_than_slot<2>(0, -1, n) != loads_younger_than_slot<2>(0, -1, 1 << 20)) { printf("prologue constant (depth 2) differs at n %d\n", n); ++bad; }
  return bad ? 1 : 0;
}
"""


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_wait_counts_equal_the_loads_behind_the_slot_in_issue_order(tmp_path):
    src = tmp_path / "counts.cpp"
    src.write_text(HARNESS)
    exe = tmp_path / "counts"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", f"-I{GEMM}", str(src), "-o", str(exe)], check=True)
    res = subprocess.run([str(exe)], capture_output=True, text=True)
    assert res.returncode == 0, res.stdout
    assert "depth 4:" in res.stdout and "depth 2:" in res.stdout and "few rows:" in res.stdout
    assert ", 0 wrong" in res.stdout.splitlines()[0]
