// Package mk.interp: the persistent role of the decode megakernel.
//
// One workgroup per CU, all resident at once.  Every workgroup walks the same instruction stream
// (MkModel.program); an instruction names an op, the op's package does this workgroup's share of it.
// Where an instruction asks for it, the workgroups meet at a grid barrier: a counter in global memory
// that only grows (barrier n is passed when it reaches n * workgroups), arrived at with an agent-scope
// release and left with an acquire, so that what one workgroup wrote (on any XCD) is what the others read.
// The wait is a bounded poll: a workgroup that gives up raises the status word and goes on, it never
// spins for ever.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "mk_device.hpp"

extern "C" __device__ void pipelink_call_op_rmsnorm(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_qkv(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_attn(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_oproj(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_upgate(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_down(const void* view, const MkInstr* instr);
extern "C" __device__ void pipelink_call_op_lmhead(const void* view, const MkInstr* instr);

namespace mk_interp {
constexpr uint32_t SPIN_LIMIT = 1u << 22;

__device__ __forceinline__ void grid_barrier(const MkModel& m, uint32_t& passed) {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");  // this wave's stores, visible device-wide
  __syncthreads();
  ++passed;
  if (threadIdx.x == 0) {
    const uint32_t target = passed * gridDim.x;
    __hip_atomic_fetch_add(m.sync, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t spin = 0;
    while ((int32_t)(__hip_atomic_load(m.sync, __ATOMIC_ACQUIRE, __HIP_MEMORY_SCOPE_AGENT) - target) < 0) {
      if (++spin >= SPIN_LIMIT) {
        __hip_atomic_fetch_or(m.sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        break;
      }
      __builtin_amdgcn_s_sleep(2);
    }
  }
  __syncthreads();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");  // nothing cached from before the barrier is read after it
}
}  // namespace mk_interp

extern "C" __device__ void mk_interp_role_worker(const void* params, unsigned variant) {
  (void)variant;
  const MkModel& m = *static_cast<const MkModel*>(params);
  const pipelink_host_view view{params, nullptr};
  uint32_t passed = 0;
  for (int i = 0; i < m.num_instr; ++i) {
    const MkInstr* instr = m.program + i;
    switch (instr->opcode) {  // uniform over the grid
      case MK_OP_RMSNORM_ATTN:
      case MK_OP_RMSNORM_FFN:
      case MK_OP_RMSNORM_FINAL: pipelink_call_op_rmsnorm(&view, instr); break;
      case MK_OP_QKV: pipelink_call_op_qkv(&view, instr); break;
      case MK_OP_ATTN: pipelink_call_op_attn(&view, instr); break;
      case MK_OP_OPROJ: pipelink_call_op_oproj(&view, instr); break;
      case MK_OP_UPGATE: pipelink_call_op_upgate(&view, instr); break;
      case MK_OP_DOWN: pipelink_call_op_down(&view, instr); break;
      case MK_OP_LMHEAD: pipelink_call_op_lmhead(&view, instr); break;
      default: break;
    }
    if (instr->barrier_after) mk_interp::grid_barrier(m, passed);
    else __syncthreads();  // the next op of this workgroup reads what this one left in LDS
  }
  // The last workgroup to get here puts the barrier counter back to zero for the next launch: by then every
  // workgroup has left its last barrier.
  if (threadIdx.x == 0) {
    const uint32_t before = __hip_atomic_fetch_add(m.sync + 2, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    if (before == gridDim.x - 1) {
      __hip_atomic_store(m.sync, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
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
#define MK_CALL(name) PL_CALL(op_##name, "op_" #name, "extern \"C\" __device__ void pipelink_call_op_" #name "(const void* view, const MkInstr* instr);")
MK_CALL(rmsnorm);
MK_CALL(qkv);
MK_CALL(attn);
MK_CALL(oproj);
MK_CALL(upgate);
MK_CALL(down);
MK_CALL(lmhead);
// the workgroup's activation vector: the normalised residual (D floats), the attention output (HQ * 64) or
// the FFN intermediate (DFF floats), whichever the running op needs; 32 KB holds DFF = 8192
PL_CLAIM("pipelink_mk_vec", "smem", 32768, 1024, "kernel");
PL_USES("pipelink_mk_vec");
PL_PRELUDE("include/mk_abi.h");
PL_EMIT_MAIN()
