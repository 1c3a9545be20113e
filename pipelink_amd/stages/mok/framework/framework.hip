// Stage package mok.framework: the persistent worker role.  It owns the schedule (which
// workgroup runs which tile, in which order) and calls the GEMM and activation owners
// through link-generated trampolines; it knows nothing of their tile internals beyond the
// published facts TILE_X / TILE_W.
//
// Plays the part of mok_framework_run in campaigns/mok/port/framework/interp_fwd.cu:26-252
// (task decode :137-214, dependency chain gate/up -> act -> down :174-213).  Not carried over: 2-CTA clusters (no
// gfx950 counterpart) and the comm clusters (single GPU).
//
// One launch runs both GEMMs (op MOK_FWD_BOTH) or one of them.  The tiles are in eight lists, one per XCD (workgroup
// id % 8): list q holds the tiles of an eighth of the routed-row tiles -- the gate/up tiles first, then the down tiles
// of the same rows; within each, expert by expert, column tile by column tile, row tiles innermost, so that
// workgroups that run at the same time share a weight tile and one XCD's L2 sees a contiguous run of experts.  A
// workgroup's first two tiles are fixed by its id; after that the list's queue (a word of the workspace) hands the
// tiles out in list order, one atomic per tile, and a workgroup whose list is handed out asks the next list's queue
// (the reference asks the cluster launch control for its next tile, interp_fwd.cu:137-160).  Tiles differ in cost
// (full ones, and those of few rows or few columns, which have a placement of their own), and turns of equal length
// leave the workgroups that drew the full ones tiles behind the others.  A down tile reads rows of `hidden` that up
// to 23 other workgroups write: it waits until the row tile's readiness counter (MokCounters) has reached the number
// of gate/up column tiles.  In every list all gate/up tiles come before the first down tile and the queue hands out
// in that order, gate/up tiles wait for nothing, and a workgroup only ever waits while it holds no unfinished tile:
// so the tiles a wait depends on are finished or running, no wait can last, and each is bounded anyway.
//
// Per workgroup the tiles are software-pipelined: the next tile's row tokens and readiness counter are requested
// behind the current tile's first loads (mok_gemm_fwd's `upcoming`), and its first loads are issued between the
// current tile's mainloop and epilogue.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "../include/mok_device.hpp"
#include "schedule.hpp"

extern "C" __device__ int pipelink_mok_fw_sched();  // byte offset of the schedule table in dynamic LDS

extern "C" __device__ void pipelink_call_gemm_init(const void* view);
extern "C" __device__ void pipelink_call_gemm_fini(const void* view);
extern "C" __device__ void pipelink_call_act_init(const void* view);
extern "C" __device__ void pipelink_call_gemm_stage(const void* view, const MokGemmTask*, const MokCounters*);
extern "C" __device__ bool pipelink_call_gemm_ready(const void* view, const MokGemmTask*, const MokCounters*);
extern "C" __device__ void pipelink_call_gemm_wait(const void* view, const MokGemmTask*, const MokCounters*);
extern "C" __device__ void pipelink_call_gemm_prefetch(const void* view, const MokGemmTask*, mok::GemmCarry*);
extern "C" __device__ void pipelink_call_gemm_fwd(const void* view, const MokGemmTask*, const MokCounters*, uint32_t*,
                                                  mok::AccFrag*, const mok::GemmCarry*, const MokGemmTask*);
extern "C" __device__ void pipelink_call_gemm_store(const void* view, const MokGemmTask*, const mok::AccFrag*);
extern "C" __device__ void pipelink_call_act_fwd(const void* view, const MokActTask*, const MokCounters*, uint32_t*,
                                                 const mok::AccFrag*);

extern "C" __device__ int pipelink_call_gemm_placement(const void* view, const MokGemmTask*);
extern "C" __device__ void pipelink_call_gemm_fwd_small(const void* view, const MokGemmTask*, const MokCounters*, uint32_t*,
                                                        mok::AccFrag*, const mok::GemmCarry*, const MokGemmTask*);
extern "C" __device__ void pipelink_call_gemm_store_small(const void* view, const MokGemmTask*, const mok::AccFrag*);
extern "C" __device__ void pipelink_call_act_fwd_small(const void* view, const MokActTask*, const MokCounters*, uint32_t*,
                                                       const mok::AccFrag*);

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mok_framework {
static_assert(TILE_X == mok::TILE_X && TILE_W == mok::TILE_W, "the schedule's tile is the GEMM owner's");

// A tile with little to multiply (mok::tile_placement): mainloop, the next tile's first loads, epilogue -- what the
// worker's loop does for a full tile, through the owners' exports for the small placement, and in a function of its
// own that is NOT inlined.  The full tile's mainloop uses every register a lane has and depends on where each value
// lives; compiled into the same function, the small tile's code takes registers from it (values kept across the tile
// loop, 100 to 270 of them spilled).  As a call it has an allocation of its own.  Everything goes in and out by value
// so that nothing of the worker's state has to live in memory.
struct SmallTileResult {
  mok::GemmCarry carry;  // of the next tile, if its prefetch was issued
  int early;             // the next tile's prefetch was issued (its rows were complete)
  uint32_t answer;       // thread 0: what the queue answered (the tile after the next)
};
__device__ __attribute__((noinline)) SmallTileResult small_tile(const void* params, MokGemmTask task, MokGemmTask next,
                                                                int32_t* counter_base, uint32_t* status, uint32_t* queue,
                                                                mok::GemmCarry carry) {
  const pipelink_host_view view{params, nullptr};
  const MokCounters counters{counter_base, status};
  // arguments travel in vector registers: say again that these are the same in every lane
  auto uniform = [](MokGemmTask& t) {
    t.op = __builtin_amdgcn_readfirstlane(t.op);
    t.expert = __builtin_amdgcn_readfirstlane(t.expert);
    t.row_begin = __builtin_amdgcn_readfirstlane(t.row_begin);
    t.row_end = __builtin_amdgcn_readfirstlane(t.row_end);
    t.col_begin = __builtin_amdgcn_readfirstlane(t.col_begin);
    t.task_idx = __builtin_amdgcn_readfirstlane(t.task_idx);
    t.counter_idx = __builtin_amdgcn_readfirstlane(t.counter_idx);
    t.wait_target = __builtin_amdgcn_readfirstlane(t.wait_target);
    t.flags = (uint32_t)__builtin_amdgcn_readfirstlane((int)t.flags);
  };
  uniform(task);
  uniform(next);
  uint32_t phase = 0;
  mok::AccFrag acc;
  pipelink_call_gemm_fwd_small(&view, &task, &counters, &phase, &acc, &carry, &next);
  uint32_t answer = 0;
  if (queue && threadIdx.x == 0) answer = __hip_atomic_fetch_add(queue, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  const bool early = next.op != 0 && pipelink_call_gemm_ready(&view, &next, &counters);
  if (early) pipelink_call_gemm_prefetch(&view, &next, &carry);
  if (task.op == MOK_GEMM_FWD_ROUTED_GATE_UP) {
    const MokActTask act{MOK_ACT_FWD_ROUTED, task.row_begin, task.row_end, task.col_begin, task.task_idx, task.counter_idx, 0u};
    pipelink_call_act_fwd_small(&view, &act, &counters, &phase, &acc);
  } else {
    pipelink_call_gemm_store_small(&view, &task, &acc);
  }
  return SmallTileResult{carry, early ? 1 : 0, answer};
}

}  // namespace mok_framework

extern "C" __device__ void mok_framework_worker(const void* params, unsigned variant) {
  (void)variant;
  using namespace mok_framework;
  const pipelink_host_view view{params, nullptr};
  const MokFrameworkParams& g = *static_cast<const MokFrameworkParams*>(params);
  Tables& tab = *reinterpret_cast<Tables*>(pipelink_smem + pipelink_mok_fw_sched());
  const int ne = g.num_experts;

  pipelink_call_gemm_init(&view);
  pipelink_call_act_init(&view);

  // exclusive prefix sums of rows and row tiles per expert (every workgroup computes its own copy)
  if (threadIdx.x == 0) tab.fill(g.tokens_per_expert, ne);
  __syncthreads();

  const Schedule sched{g, tab, tab.tile_begin[ne], g.op == MOK_GEMM_FWD_ROUTED_DOWN ? 0 : g.num_col_tiles_gate_up,
                       g.op == MOK_GEMM_FWD_ROUTED_GATE_UP ? 0 : g.num_col_tiles_down};
  const MokCounters counters{g.op == MOK_FWD_BOTH ? reinterpret_cast<int32_t*>(g.workspace + MOK_WS_COUNTERS) : nullptr,
                             g.workspace + MOK_WS_STATUS};
  uint32_t phase = 0;

  const int q = blockIdx.x % NUM_XCD;
  const int turn = gridDim.x / NUM_XCD;  // the launch grid is a multiple of NUM_XCD: workgroups per list
  const int items = sched.length(q);
  int i = blockIdx.x / NUM_XCD, cursor = 0;
  if (i < items) {
    MokGemmTask task = sched.decode(q, i, cursor);
    // the first tile has no mainloop in front of it to look ahead from
    pipelink_call_gemm_stage(&view, &task, &counters);
    __syncthreads();  // waits for the staged loads, then the barrier
    if (!pipelink_call_gemm_ready(&view, &task, &counters)) pipelink_call_gemm_wait(&view, &task, &counters);
    mok::GemmCarry carry;
    pipelink_call_gemm_prefetch(&view, &task, &carry);
    // The tile after this one: the workgroup's second turn.  From there on tiles are handed out by the list's queue (a
    // counter in the workspace), one request per tile, made while the tile before the one before is multiplied: tiles
    // differ in cost (full ones, and those with few rows or few columns), and turns of equal length would leave the
    // workgroups that drew the full ones behind the others by several tiles' time.
    // A workgroup whose list has been handed out goes on with the next list's queue (and so on, once round): the
    // lists are cut by number of tiles, not by cost, and whole XCDs would otherwise end a tile or two before others.
    int list = q;   // the list this workgroup asks
    int tried = 1;  // lists it has asked so far
    MokGemmTask next = task;
    if (i + turn < items) next = sched.decode(q, i + turn, cursor);
    else next.op = 0;  // no task: mok_gemm_fwd looks ahead to nothing
    for (;;) {
      const bool has_next = next.op != 0;
      const bool asks = has_next && tried <= NUM_XCD;  // (a workgroup that has found every list handed out asks no more)
      uint32_t answer = 0;
      bool early;
      if (pipelink_call_gemm_placement(&view, &task) != mok::TILE_FULL) {
        const SmallTileResult res = small_tile(params, task, next, counters.base, counters.status, asks ? g.workspace + MOK_WS_QUEUE + list : nullptr, carry);
        carry = res.carry;
        early = __builtin_amdgcn_readfirstlane(res.early) != 0;
        answer = res.answer;
        ++phase;
      } else {
        mok::AccFrag acc;
        pipelink_call_gemm_fwd(&view, &task, &counters, &phase, &acc, &carry, &next);
        // ask the queue for the tile after the next (one thread); the answer has the epilogue's time to arrive
        if (asks && threadIdx.x == 0)
          answer = __hip_atomic_fetch_add(g.workspace + MOK_WS_QUEUE + list, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        // The next tile's first loads fly while this tile's epilogue computes -- unless its rows are not complete yet:
        // then this tile is finished (and counted) first, so that nobody waits for a workgroup that waits.
        early = has_next && pipelink_call_gemm_ready(&view, &next, &counters);
        if (early) pipelink_call_gemm_prefetch(&view, &next, &carry);
        if (task.op == MOK_GEMM_FWD_ROUTED_GATE_UP) {
          const MokActTask act{MOK_ACT_FWD_ROUTED, task.row_begin, task.row_end, task.col_begin, task.task_idx, task.counter_idx, 0u};
          pipelink_call_act_fwd(&view, &act, &counters, &phase, &acc);
        } else {
          pipelink_call_gemm_store(&view, &task, &acc);
        }
      }
      // the queue's answer goes round the workgroup through LDS; the barrier is one every wave reaches at about the
      // same time (the epilogue has just ended with one)
      if (threadIdx.x == 0) tab.claim = answer;
      mok::lds_barrier();
      MokGemmTask after = next;
      after.op = 0;
      if (asks) {
        int k = 2 * turn + (int)tab.claim;
        while (k >= sched.length(list) && tried < NUM_XCD) {
          // this list has been handed out: ask the next one, and wait for the answer (at a launch's end only)
          list = list + 1 == NUM_XCD ? 0 : list + 1;
          ++tried;
          mok::lds_barrier();  // everybody has read the last answer
          if (threadIdx.x == 0)
            tab.claim = __hip_atomic_fetch_add(g.workspace + MOK_WS_QUEUE + list, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          mok::lds_barrier();
          k = 2 * turn + (int)tab.claim;
        }
        if (k < sched.length(list)) after = sched.decode(list, k, cursor);
        else tried = NUM_XCD + 1;  // every list has been handed out
      }
      if (!has_next) break;
      if (!early) {
        pipelink_call_gemm_wait(&view, &next, &counters);
        pipelink_call_gemm_prefetch(&view, &next, &carry);
      }
      task = next;
      next = after;
    }
  }
  pipelink_call_gemm_fini(&view);

  // The last workgroup to leave puts the queues and the counters back to zero for the next launch: by then nobody
  // asks or waits any more.
  if (threadIdx.x == 0) {
    const uint32_t before = __hip_atomic_fetch_add(g.workspace + MOK_WS_FINISHED, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    tab.last = before == gridDim.x - 1 ? 1u : 0u;
  }
  __syncthreads();
  if (tab.last) {
    if (g.op == MOK_FWD_BOTH)
      for (int w = threadIdx.x; w < sched.row_tiles; w += blockDim.x)
        __hip_atomic_store(g.workspace + MOK_WS_COUNTERS + w, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (threadIdx.x < NUM_XCD) __hip_atomic_store(g.workspace + MOK_WS_QUEUE + threadIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (threadIdx.x == 0) {
      __hip_atomic_store(g.workspace + MOK_WS_FINISHED, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(g.workspace + MOK_WS_GAVE_UP, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}
#else  // PIPELINK_EMIT: host-evaluated annotations only
#include "../include/mok_abi.h"
#endif

PL_STAGE("mok.framework", "0.2.0");
PL_PARAMS(MokFrameworkParams);
PL_ROLE(worker, mok_framework_worker, 4);
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_CALL(gemm_init, "mok_gemm_init", "extern \"C\" __device__ void pipelink_call_gemm_init(const void* view);");
PL_CALL(gemm_fini, "mok_gemm_fini", "extern \"C\" __device__ void pipelink_call_gemm_fini(const void* view);");
PL_CALL(act_init, "mok_act_init", "extern \"C\" __device__ void pipelink_call_act_init(const void* view);");
PL_CALL(gemm_stage, "mok_gemm_stage",
        "extern \"C\" __device__ void pipelink_call_gemm_stage(const void* view, const MokGemmTask* task, const MokCounters* counters);");
PL_CALL(gemm_ready, "mok_gemm_ready",
        "extern \"C\" __device__ bool pipelink_call_gemm_ready(const void* view, const MokGemmTask* task, const MokCounters* counters);");
PL_CALL(gemm_wait, "mok_gemm_wait",
        "extern \"C\" __device__ void pipelink_call_gemm_wait(const void* view, const MokGemmTask* task, const MokCounters* counters);");
PL_CALL(gemm_prefetch, "mok_gemm_prefetch",
        "extern \"C\" __device__ void pipelink_call_gemm_prefetch(const void* view, const MokGemmTask* task, mok::GemmCarry* carry);");
PL_CALL(gemm_fwd, "mok_gemm_fwd",
        "extern \"C\" __device__ void pipelink_call_gemm_fwd(const void* view, const MokGemmTask* task, "
        "const MokCounters* counters, uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry, "
        "const MokGemmTask* upcoming);");
PL_CALL(gemm_store, "mok_gemm_store",
        "extern \"C\" __device__ void pipelink_call_gemm_store(const void* view, const MokGemmTask* task, const mok::AccFrag* acc);");
PL_CALL(act_fwd, "mok_act_fwd",
        "extern \"C\" __device__ void pipelink_call_act_fwd(const void* view, const MokActTask* task, "
        "const MokCounters* counters, uint32_t* phase, const mok::AccFrag* acc);");
PL_CALL(gemm_placement, "mok_gemm_placement",
        "extern \"C\" __device__ int pipelink_call_gemm_placement(const void* view, const MokGemmTask* task);");
PL_CALL(gemm_fwd_small, "mok_gemm_fwd_small",
        "extern \"C\" __device__ void pipelink_call_gemm_fwd_small(const void* view, const MokGemmTask* task, "
        "const MokCounters* counters, uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry, "
        "const MokGemmTask* upcoming);");
PL_CALL(gemm_store_small, "mok_gemm_store_small",
        "extern \"C\" __device__ void pipelink_call_gemm_store_small(const void* view, const MokGemmTask* task, const mok::AccFrag* acc);");
PL_CALL(act_fwd_small, "mok_act_fwd_small",
        "extern \"C\" __device__ void pipelink_call_act_fwd_small(const void* view, const MokActTask* task, "
        "const MokCounters* counters, uint32_t* phase, const mok::AccFrag* acc);");
// schedule tables: exclusive prefix sums of rows and row tiles for up to 256 experts, and one word more
PL_CLAIM("pipelink_mok_fw_sched", "smem", 2 * (256 + 1) * 4 + 8, 16, "kernel");
PL_USES("pipelink_mok_fw_sched");
// host contract: the schedule's owner
PL_HOST_GROUP("mok.framework.params", "mok_framework");
PL_HOST_ABI_TYPE(3, MokFrameworkParams);
MOK_HOST_SCALARS();
PL_HOST_CHANNEL(1, "tokens_per_expert", 32, "read", "mok.num_local_experts", false);
// status word and readiness counters of a launch: all zero before the first launch, every launch leaves them zero
PL_HOST_CHANNEL(2, "workspace", 32, "write", "mok.workspace_words", false);
PL_FACT("mok.framework.MAX_EXPERTS", 256);
PL_FACT("mok.framework.LISTS", 8);
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
