// Device side of a produce/consume ring in LDS on gfx950.
//
// The reference's rings are driven by hardware mbarrier objects (arrive counts, transaction
// bytes, phase bits; examples/ring-pipeline/src/{producer,consumer}.cu).  CDNA4 has no such
// object.  Here a ring stage has two 32-bit counters in LDS, one 16-byte slot each in the
// "mbarrier" claim domain, that only ever grow:
//   full[i]   counts producer arrivals: stage i has been filled  floor(full[i] / arrive_full)  times
//   empty[i]  counts consumer arrivals: stage i has been drained floor(empty[i] / arrive_empty) times
// The consumer's n-th use of a stage (n = 0, 1, ...) waits for full >= (n + 1) * arrive_full; the
// producer's n-th fill waits for empty >= n * arrive_empty.  The dispatch kernel zeroes the
// counters before any role starts (the manifest's init.materializer = "dispatch").
//
// Ordering.  LDS operations of one wave execute in order, and a wave's global->LDS loads have
// written LDS when its vmcnt says they are done.  So a producer arrives with s_waitcnt vmcnt(N)
// followed by a plain LDS atomic add (no fence: a fence would wait for every load in flight and
// serialise the ring), and a consumer that has seen the count may read the stage.  A consumer
// arrives on `empty` after s_waitcnt lgkmcnt(0): its reads have returned.
//
// Waits are bounded: after `spin_limit` polls the wait gives up and returns false, so a protocol
// bug ends as a wrong result and a raised flag, never as a wave that spins for ever.
#ifndef PIPELINK_RING_HPP
#define PIPELINK_RING_HPP

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pl {

constexpr uint32_t RING_SPIN_LIMIT = 1u << 22;

// counter i of the ring whose first 16-byte slot index is `base_slot` (a solved handle)
__device__ __forceinline__ uint32_t* ring_counter(unsigned char* smem, int base_slot, int i) {
  return reinterpret_cast<uint32_t*>(smem + 16 * (base_slot + i));
}

// polls until *counter >= target (wrap-safe); false if it gave up
__device__ __forceinline__ bool ring_wait(uint32_t* counter, uint32_t target, uint32_t spin_limit = RING_SPIN_LIMIT) {
  for (uint32_t spin = 0; spin < spin_limit; ++spin) {
    const uint32_t seen = __hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    if ((int32_t)(seen - target) >= 0) {
      asm volatile("" ::: "memory");  // nothing that reads the stage moves above the poll
      return true;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  return false;
}

// one arrival by the calling wave (call it from one lane)
__device__ __forceinline__ void ring_arrive(uint32_t* counter) {
  asm volatile("" ::: "memory");
  __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// s_waitcnt vmcnt(n): at most n of this wave's global loads still in flight (n < 64)
template <int N>
__device__ __forceinline__ void ring_wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
  asm volatile("" ::: "memory");
}
// s_waitcnt lgkmcnt(0): this wave's LDS reads have returned
__device__ __forceinline__ void ring_wait_reads() {
  __builtin_amdgcn_s_waitcnt(0xC07F);
  asm volatile("" ::: "memory");
}

}  // namespace pl

#endif
