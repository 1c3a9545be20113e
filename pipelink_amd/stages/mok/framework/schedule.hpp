// The MoK framework stage's schedule: which tiles a launch has, in which of the eight lists, in which order, and
// item -> task.  Plain C++ on plain integers, so that a host compiler takes it too: the tests enumerate the lists on
// the CPU (every tile of both GEMMs exactly once, gate/up tiles before down tiles, row and column ranges) with
// MOK_SCHED_FN defined empty and MOK_SCHED_UNIFORM(x) as x.
//
// Plays the part of the task decode in campaigns/mok/port/framework/interp_fwd.cu:137-214.
#ifndef PIPELINK_MOK_FRAMEWORK_SCHEDULE_HPP
#define PIPELINK_MOK_FRAMEWORK_SCHEDULE_HPP
#include <stdint.h>
#include "../include/mok_abi.h"

#ifndef MOK_SCHED_FN
#define MOK_SCHED_FN __device__ __forceinline__
// wave-uniform by construction; say so, so that the value lives in a scalar register
#define MOK_SCHED_UNIFORM(x) __builtin_amdgcn_readfirstlane(x)
#endif

namespace mok_framework {
constexpr int MAX_EXPERTS = 256;
constexpr int NUM_XCD = 8;       // lists
constexpr int TILE_X = 256;      // routed rows of a tile   (the GEMM owner's published facts; the stage source
constexpr int TILE_W = 256;      // weight rows of a tile    checks them against the owner's header)

// the schedule's tables in LDS: exclusive prefix sums per expert, and one word of the last workgroup
struct Tables {
  int row_begin[MAX_EXPERTS + 1];
  int tile_begin[MAX_EXPERTS + 1];
  uint32_t last;   // 1 in the workgroup that leaves the launch last
  uint32_t claim;  // what the list's queue answered this workgroup's last request

  // exclusive prefix sums of rows and row tiles per expert (one thread; every workgroup computes its own copy)
  MOK_SCHED_FN void fill(const int32_t* tokens_per_expert, int ne) {
    int rows = 0, tiles = 0;
    for (int e = 0; e < ne; ++e) {
      row_begin[e] = rows;
      tile_begin[e] = tiles;
      const int c = tokens_per_expert[e];
      rows += c;
      tiles += (c + TILE_X - 1) / TILE_X;
    }
    row_begin[ne] = rows;
    tile_begin[ne] = tiles;
  }
};

struct Schedule {
  const MokFrameworkParams& g;
  const Tables& tab;
  int row_tiles;  // of all experts
  int gate_up_cols, down_cols;  // column tiles of the GEMMs this launch runs (0: not run)

  // List q: the q-th eighth of the gate/up tiles (all experts' tiles in one sequence: expert by expert, column tile by
  // column tile, row tiles innermost), then the q-th eighth of the down tiles.
  MOK_SCHED_FN int share(int q, int total) const { return (int)((long long)q * total / NUM_XCD); }
  MOK_SCHED_FN int length(int q) const {
    const int gu = row_tiles * gate_up_cols, d = row_tiles * down_cols;
    return share(q + 1, gu) - share(q, gu) + share(q + 1, d) - share(q, d);
  }

  // item i of list q -> task.  `cursor` is the expert of the item this workgroup decoded last: a workgroup's items
  // come in growing order as long as it stays in one GEMM, so the search usually ends where it starts.
  MOK_SCHED_FN MokGemmTask decode(int q, int i, int& cursor) const {
    const int gu = row_tiles * gate_up_cols, d = row_tiles * down_cols;
    const int gate_up_items = share(q + 1, gu) - share(q, gu);
    const bool gate_up = i < gate_up_items;
    const int idx = gate_up ? share(q, gu) + i : share(q, d) + i - gate_up_items;  // in the sequence of its GEMM's tiles
    const int cols = gate_up ? gate_up_cols : down_cols;
    // last e with tile_begin[e] * cols <= idx: it has row tiles, since tile_begin[e + 1] * cols > idx
    int lo = cursor;
    if (tab.tile_begin[lo] * cols > idx) lo = 0;  // the other GEMM: from the start
    while (lo + 1 < g.num_experts && tab.tile_begin[lo + 1] * cols <= idx) ++lo;
    cursor = lo;
    const int e = MOK_SCHED_UNIFORM(lo);
    const int t0 = tab.tile_begin[e], t1 = tab.tile_begin[e + 1];
    const int local = idx - t0 * cols;
    const int col = local / (t1 - t0);
    const int tile = t0 + local - col * (t1 - t0);  // row tile, counted over all experts
    const int first = tab.row_begin[e] + (tile - tab.tile_begin[e]) * TILE_X;
    const bool both = g.op == MOK_FWD_BOTH;
    // wave-uniform by construction; say so, so that the task lives in scalar registers
    MokGemmTask t;
    t.op = gate_up ? MOK_GEMM_FWD_ROUTED_GATE_UP : MOK_GEMM_FWD_ROUTED_DOWN;
    t.expert = e;
    t.row_begin = MOK_SCHED_UNIFORM(first);
    t.row_end = MOK_SCHED_UNIFORM(tab.row_begin[e + 1]);
    t.col_begin = MOK_SCHED_UNIFORM(col * (gate_up ? TILE_W / 2 : TILE_W));
    t.task_idx = MOK_SCHED_UNIFORM(q << 24 | i);
    t.counter_idx = MOK_SCHED_UNIFORM(both ? tile : -1);
    t.wait_target = gate_up ? 0 : gate_up_cols;
    t.flags = 0u;
    return t;
  }
};

}  // namespace mok_framework

#endif
