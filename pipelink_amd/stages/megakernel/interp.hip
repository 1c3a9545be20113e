// Package mk.interp: the persistent role of the decode megakernel.
//
// One workgroup per CU, all resident at once.  Every workgroup walks the same instruction stream
// (MkModel.program); an instruction names an op, the op's package does this workgroup's share of it.
// Where an instruction asks for it, the workgroups meet at a grid barrier: counters in global memory that
// grow through the launch, so that what one workgroup wrote (on any XCD) before it is what the others read after it.
// The barrier is in two halves.  A workgroup arrives as soon as its op is done and goes on into the next op, which
// first asks memory for what no workgroup writes (its first rows of weights, its stretch of the cache) and only
// then calls back (channel inputs_<op>) to wait for the others: the barrier's 2.5 us and the first loads' latency
// run side by side.  A normalisation instruction is held back in the same way and runs inside that call.
// The wait is a bounded poll: a workgroup that gives up raises the status word and goes on; a launch never spins
// for ever, and one that cannot complete its barriers ends in well under a second.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_op_rmsnorm(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_qkv(const void* view, const MkInstr* instr, MkPending* pending);
extern "C" __device__ void pipelink_call_op_attn(const void* view, const MkInstr* instr, MkPending* pending);
extern "C" __device__ void pipelink_call_op_oproj(const void* view, const MkInstr* instr, MkPending* pending);
extern "C" __device__ void pipelink_call_op_upgate(const void* view, const MkInstr* instr, MkPending* pending);
extern "C" __device__ void pipelink_call_op_down(const void* view, const MkInstr* instr, MkPending* pending);
extern "C" __device__ void pipelink_call_op_lmhead(const void* view, const MkInstr* instr, MkPending* pending);

// the opcode numbers the link bound to the op packages' claims
extern "C" __device__ int pipelink_mk_opcode_rmsnorm_attn();
extern "C" __device__ int pipelink_mk_opcode_qkv();
extern "C" __device__ int pipelink_mk_opcode_attn();
extern "C" __device__ int pipelink_mk_opcode_oproj();
extern "C" __device__ int pipelink_mk_opcode_rmsnorm_ffn();
extern "C" __device__ int pipelink_mk_opcode_upgate();
extern "C" __device__ int pipelink_mk_opcode_down();
extern "C" __device__ int pipelink_mk_opcode_rmsnorm_final();
extern "C" __device__ int pipelink_mk_opcode_lmhead();

namespace mk_interp {
// A wait that is not answered within this many polls is given up.  A barrier takes about 2.5 us, a poll a fraction of a
// microsecond to a microsecond: 2^13 polls are 5 to 8 ms, two thousand barriers' worth.  A launch whose barriers cannot
// complete (more workgroups than can be resident, CUs held by another process) gives up each of its 80 waits after
// that long and ends, with its status word raised, in well under a second.  Making the first give-up final for the
// workgroup would end it sooner, but every way of remembering it across the ops -- a field of MkPending, a bit of its
// barrier word, a note in LDS consulted in the poll loop, a look at the status word every 256 polls -- made the step
// 6 to 25 us slower (the ops have no register to spare, and the poll loop no instruction), so the bound is kept by
// the limit alone.
constexpr uint32_t SPIN_LIMIT = 1u << 13;
constexpr uint32_t STATUS_GAVE_UP = 1u;

// Arrival and release are both in two levels.  An atomic or a load that every XCD must agree on is performed at
// the memory side, one after the other: 256 of them on one word cost more than the work between two barriers.
// So a workgroup first arrives on its XCD's own counter (workgroups are dealt to the 8 XCDs round-robin,
// blockIdx % 8; an access at workgroup scope is served by that XCD's L2), and only the last arrival of an XCD
// goes on to the grid's counter.  One workgroup per XCD polls the grid's counter and then passes the word on to
// its XCD in a generation number the others poll in their L2.  No cache is written back or invalidated here: what
// workgroups hand each other across a barrier is stored and loaded at device scope (mk::shared_store / shared_load),
// and every wave has waited for its stores (the __syncthreads) before its workgroup is counted.
//
// Counters grow through a launch (barrier g of the launch is generation g) and are put back to zero at its end by
// whoever may touch them: every word is only ever accessed at one scope.  An XCD's words (arrivals, generation,
// finished) are accessed at workgroup scope by that XCD's workgroups, and the last of them to finish zeroes them;
// the grid's words at device scope, and the last workgroup of the grid zeroes those.  So a launch needs no memset
// and no word is ever written from two scopes (a device-scope store to a word that another XCD's L2 holds modified
// could be undone by that line's write-back).
//
// The round-robin assumption is recorded, not trusted blindly: in a session's first launch (sync[3] still zero) every
// workgroup stores the XCC it really runs on (hardware register XCC_ID) into a word of its own, sync[512 + blockIdx];
// the host checks that the workgroups with one blockIdx % 8 all ran on one XCC and no two such groups on the same
// (host/megakernel.py raise_on_status).  (One word per workgroup, a plain store, one launch: 256 device-scope atomics
// on one line in every launch cost 8 us per token.)
constexpr int NUM_XCD = 8;
constexpr int XCD_COUNTER = 32;      // sync[32 * (1 + xcd)]: arrivals; [.. + 1]: generation; [.. + 2]: finished; one 128-byte line per XCD
constexpr int XCC_SEEN = 512;        // sync[512 + blockIdx]: XCC_RECORDED | the XCC that workgroup ran on
constexpr int XCC_WORDS = 512;
constexpr uint32_t XCC_RECORDED = 0x100u;
// false: the wait was given up (the status word is raised then; it is sticky, the host clears it).  The loop looks at
// nothing but the word it waits for: a look at the status word as well, even one in 256 polls, cost 6-11 us per token.
__device__ __forceinline__ bool poll(uint32_t* word, uint32_t target, bool local, const MkModel& m) {
  for (uint32_t spin = 0; spin < SPIN_LIMIT; ++spin) {
    // local: an atomic add of 0 written out as such -- atomics are performed in the L2, whereas a plain
    // workgroup-scope load (which the compiler makes of an idempotent read-modify-write) could be served by
    // this CU's L1 for ever
    uint32_t seen;
    if (local) {
      const uint32_t zero = 0;
      asm volatile("global_atomic_add %0, %1, %2, off sc0\n\ts_waitcnt vmcnt(0)" : "=&v"(seen) : "v"(word), "v"(zero) : "memory");
    } else {
      // two loads in flight, a fraction of a round trip apart: the answer is half a round trip old on average, not a whole one
      seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_s_sleep(4);
      const uint32_t later = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if ((int32_t)(seen - target) >= 0) return true;
      seen = later;
    }
    if ((int32_t)(seen - target) >= 0) return true;
    __builtin_amdgcn_s_sleep(1);
  }
  __hip_atomic_fetch_or(m.sync + 1, STATUS_GAVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  return false;
}
// first half of barrier number `generation` (1, 2, ...) of the launch: this workgroup has finished what comes before it
__device__ __forceinline__ void grid_arrive(const MkModel& m, uint32_t generation) {
  // Every wave first waits until its own stores have been written through (a store leaves the wave's vector-memory
  // count when it is acknowledged; the barrier's workgroup-scope fence does not wait for that): what the workgroup hands
  // the others is in memory before it says that it has arrived.
  __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t xcd = blockIdx.x % NUM_XCD;
    const uint32_t members = (gridDim.x - xcd + NUM_XCD - 1) / NUM_XCD;
    const uint32_t before = __hip_atomic_fetch_add(m.sync + XCD_COUNTER * (1 + xcd), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if (before + 1 == generation * members)
      __hip_atomic_fetch_add(m.sync, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}
// second half: every workgroup has arrived at barrier number pending->barrier.  The wait is bounded by SPIN_LIMIT polls
// and nothing else: a workgroup that has given up one barrier polls the next one again for as long (keeping "gave up
// once" across the ops was measured and costs more than it saves, see SPIN_LIMIT), so a launch that cannot complete
// pays up to SPIN_LIMIT polls per barrier and workgroup.  (A workgroup that was not running finds every barrier
// complete when it gets there, because arrivals go on.)
__device__ __forceinline__ void grid_wait(const MkModel& m, MkPending* pending) {
  const uint32_t generation = pending->barrier;
  if (threadIdx.x == 0) {
    const uint32_t xcd = blockIdx.x % NUM_XCD, groups = min((uint32_t)NUM_XCD, gridDim.x);
    uint32_t* mine = m.sync + XCD_COUNTER * (1 + xcd);
    if (blockIdx.x < NUM_XCD) {  // this XCD's first workgroup listens for the grid
      poll(m.sync, generation * groups, false, m);
      __hip_atomic_exchange(mine + 1, generation, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    } else {
      poll(mine + 1, generation, true, m);
    }
  }
  pending->barrier = 0;
  __syncthreads();
}
}  // namespace mk_interp

// The ops' way to their inputs: the open barrier, then the normalisation that is due.
__device__ __forceinline__ void mk_interp_inputs(const void* view, MkPending* pending) {
  const MkModel& m = *static_cast<const MkModel*>(static_cast<const pipelink_host_view*>(view)->residue);
  if (pending->barrier != 0) mk_interp::grid_wait(m, pending);
  if (pending->norm != nullptr) {
    pipelink_call_op_rmsnorm(view, pending->norm);
    pending->norm = nullptr;
    __syncthreads();  // the op reads what the normalisation left in LDS
  }
}

// a channel has one caller: one export per op package
#define MK_INPUTS(name) \
  extern "C" __device__ void mk_interp_inputs_##name(const void* view, MkPending* pending) { mk_interp_inputs(view, pending); }
MK_INPUTS(qkv)
MK_INPUTS(attn)
MK_INPUTS(oproj)
MK_INPUTS(upgate)
MK_INPUTS(down)
MK_INPUTS(lmhead)
#undef MK_INPUTS

extern "C" __device__ void mk_interp_role_worker(const void* params, unsigned variant) {
  (void)variant;
  const MkModel& m = *static_cast<const MkModel*>(params);
  const pipelink_host_view view{params, nullptr};
  uint32_t passed = 0;
  MkPending pending{nullptr, 0};
  if (threadIdx.x == 0 && blockIdx.x < mk_interp::XCC_WORDS &&
      __hip_atomic_load(m.sync + 3, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) == 0) {
    // the session's first launch records where its workgroups run (the dispatch pattern does not change from launch
    // to launch).  XCC_ID is bits 3:0 of hardware register 20: s_getreg_b32 with size 4, offset 0
    const uint32_t xcc = (uint32_t)__builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xFu;
    __hip_atomic_store(m.sync + mk_interp::XCC_SEEN + blockIdx.x, mk_interp::XCC_RECORDED | xcc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  for (int i = 0; i < m.num_instr; ++i) {
    const MkInstr* instr = m.program + i;
    const int op = instr->opcode;  // uniform over the grid; the numbers are bound at link time
    const bool norm = op == pipelink_mk_opcode_rmsnorm_attn() || op == pipelink_mk_opcode_rmsnorm_ffn() || op == pipelink_mk_opcode_rmsnorm_final();
    if (norm && pending.norm == nullptr && !instr->barrier_after) {
      pending.norm = instr;  // runs when the next op asks for its inputs: that op's first loads are on their way by then
      continue;
    }
    if (norm) {
      mk_interp_inputs(&view, &pending);
      pipelink_call_op_rmsnorm(&view, instr);
    } else if (op == pipelink_mk_opcode_qkv()) pipelink_call_op_qkv(&view, instr, &pending);
    else if (op == pipelink_mk_opcode_attn()) pipelink_call_op_attn(&view, instr, &pending);
    else if (op == pipelink_mk_opcode_oproj()) pipelink_call_op_oproj(&view, instr, &pending);
    else if (op == pipelink_mk_opcode_upgate()) pipelink_call_op_upgate(&view, instr, &pending);
    else if (op == pipelink_mk_opcode_down()) pipelink_call_op_down(&view, instr, &pending);
    else if (op == pipelink_mk_opcode_lmhead()) pipelink_call_op_lmhead(&view, instr, &pending);
    mk_interp_inputs(&view, &pending);  // an opcode nobody claimed, or an op that had nothing to do
    if (instr->barrier_after) {
      mk_interp::grid_arrive(m, ++passed);
      pending.barrier = passed;
    } else {
      __syncthreads();  // the next op of this workgroup reads what this one left in LDS
    }
  }
  mk_interp_inputs(&view, &pending);
  // Every workgroup has left its last barrier of the launch when it gets here (it arrives at every barrier, waited for
  // or not, so the counts are whole even after a give-up).  The last of an XCD's workgroups puts that XCD's words back
  // to zero, the last of the grid the grid's words: each at the scope the words are used at.
  if (threadIdx.x == 0) {
    const uint32_t xcd = blockIdx.x % mk_interp::NUM_XCD;
    const uint32_t members = (gridDim.x - xcd + mk_interp::NUM_XCD - 1) / mk_interp::NUM_XCD;
    uint32_t* mine = m.sync + mk_interp::XCD_COUNTER * (1 + xcd);
    if (__hip_atomic_fetch_add(mine + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) == members - 1) {
      __hip_atomic_store(mine, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_store(mine + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      __hip_atomic_store(mine + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    const uint32_t before = __hip_atomic_fetch_add(m.sync + 2, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    if (before == gridDim.x - 1) {
      __hip_atomic_store(m.sync, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_fetch_add(m.sync + 3, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // launches closed
      __hip_atomic_store(m.sync + 2, 0u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}
#else
#include "include/mk_abi.h"
#endif

PL_STAGE("mk.interp", "0.1.0");
PL_PARAMS(MkModel);
PL_ROLE(worker, mk_interp_role_worker, 4);
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {});
PL_CALL(op_rmsnorm, "op_rmsnorm", "extern \"C\" __device__ void pipelink_call_op_rmsnorm(const void* view, const MkInstr* instr);");
#define MK_CALL(name) \
  PL_CALL(op_##name, "op_" #name, "extern \"C\" __device__ void pipelink_call_op_" #name "(const void* view, const MkInstr* instr, MkPending* pending);")
MK_CALL(qkv);
MK_CALL(attn);
MK_CALL(oproj);
MK_CALL(upgate);
MK_CALL(down);
MK_CALL(lmhead);
// what an op calls once before it reads its inputs (MkPending in include/mk_abi.h)
#define MK_SERVE_INPUTS(name)                                                                                                      \
  PL_EXPORT(inputs_##name, mk_interp_inputs_##name, "extern \"C\" __device__ void mk_interp_inputs_" #name "(const void* view, MkPending* pending);"); \
  PL_SERVE(inputs_##name, "inputs_" #name)
MK_SERVE_INPUTS(qkv);
MK_SERVE_INPUTS(attn);
MK_SERVE_INPUTS(oproj);
MK_SERVE_INPUTS(upgate);
MK_SERVE_INPUTS(down);
MK_SERVE_INPUTS(lmhead);
// the workgroup's activation vector: the normalised residual (D floats), the attention output (HQ * 64) or
// the FFN intermediate (DFF floats), whichever the running op needs; 32 KB holds DFF = 8192, and 1 KB behind it is
// the ops' reduction scratch
PL_CLAIM("pipelink_mk_vec", "smem", 33792, 1024, "kernel");
PL_USES("pipelink_mk_vec");
PL_USES("pipelink_mk_opcode_rmsnorm_attn");
PL_USES("pipelink_mk_opcode_qkv");
PL_USES("pipelink_mk_opcode_attn");
PL_USES("pipelink_mk_opcode_oproj");
PL_USES("pipelink_mk_opcode_rmsnorm_ffn");
PL_USES("pipelink_mk_opcode_upgate");
PL_USES("pipelink_mk_opcode_down");
PL_USES("pipelink_mk_opcode_rmsnorm_final");
PL_USES("pipelink_mk_opcode_lmhead");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
