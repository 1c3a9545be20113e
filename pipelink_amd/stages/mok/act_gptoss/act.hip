// Owner package mok.act (GPT-OSS flavour): clamped SwiGLU with alpha = 1.702 applied to
// the gate/up accumulator of one tile, rounded to bf16, then requantised to MXFP8 along
// the d_ff axis (one e8m0 scale per 32 columns of a routed row).
//
// Replaces swiglu_fwd_kernel<false, IS_CLAMPED> of
// campaigns/mok/port/act_gptoss/swiglu.cuh:45-217 (MXFP8 branch :157-195).  Differences by
// design: the inputs arrive as fp32 MFMA accumulators instead of bf16 tiles read back
// from HBM, and only the row-wise (forward) quantised copy is written.
//
// The body only uses the placement contract of mok::AccFrag (which routed row and column
// a (fragment, register, lane) triple is); it does not care whether the GEMM owner kept
// the accumulator in AGPRs, VGPRs or LDS.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "../include/mok_device.hpp"

extern "C" __device__ int pipelink_mok_clamp();      // link-time variant: 1 = clamp to +-limit
extern "C" __device__ int pipelink_mok_act_arena();  // byte offset of the staging tile in dynamic LDS

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mok_act_owner {
using namespace mok;

constexpr float SWIGLU_ALPHA = 1.702f;  // campaigns/mok/port/act_gptoss/swiglu.cuh:2
constexpr int STAGE_PITCH = TILE_W / 2 + 16;            // bytes per staged row: 128 codes + pad against bank conflicts
constexpr int STAGE_SCALE_OFF = TILE_X * STAGE_PITCH;   // [row][4] scale bytes behind the codes

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

// v_min_f32 as written: fminf() first quiets a signalling NaN with an extra instruction per
// element, which an MFMA accumulator cannot hold
__device__ __forceinline__ float min_raw(float a, float b) {
  float r;
  asm("v_min_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
  return r;
}

template <bool CLAMPED>
__device__ __forceinline__ float swiglu(float gate, float up, float limit) {
  if (CLAMPED) {
    gate = min_raw(gate, limit);
    up = __builtin_amdgcn_fmed3f(up, -limit, limit);
  }
  // (up + 1) * gate * sigmoid(alpha * gate) with the hardware exp2 and reciprocal, as in the
  // reference's --use_fast_math build (campaigns/mok/port/build.py:26)
  const float den = 1.0f + __builtin_amdgcn_exp2f(gate * (-SWIGLU_ALPHA * 1.4426950408889634f));
  return (up + 1.0f) * (gate * __builtin_amdgcn_rcpf(den));
}

typedef short s16x2 __attribute__((ext_vector_type(2)));
typedef unsigned int u32x4 __attribute__((__vector_size__(16)));

// Four floats -> four e4m3 codes of a block whose scale is `scale` (a power of two): round to
// bf16 (nearest even, v_cvt_pk_bf16_f32: the reference rounds to bf16 before quantising,
// swiglu.cuh:175), divide by the scale and round to e4m3 (v_cvt_scalef32_pk_fp8_bf16, nearest
// even, exact division).  That conversion does not saturate (a quotient above 448 becomes NaN),
// so the floats are first clamped to +-448 * scale; the bound is a bf16 number, so clamping
// before the bf16 rounding gives what clamping after it would (measured against the separate
// multiply / clamp / v_cvt_pk_fp8_f32 sequence over a sweep of mantissas, exponents and scales).
__device__ __forceinline__ uint32_t quantise4(float a, float b, float c, float d, float limit, float scale) {
  const f32x2 lo = {__builtin_amdgcn_fmed3f(a, -limit, limit), __builtin_amdgcn_fmed3f(b, -limit, limit)};
  const f32x2 hi = {__builtin_amdgcn_fmed3f(c, -limit, limit), __builtin_amdgcn_fmed3f(d, -limit, limit)};
  s16x2 v = {0, 0};
  v = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(v, __builtin_convertvector(lo, bf16x2), scale, false);
  v = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(v, __builtin_convertvector(hi, bf16x2), scale, true);
  return __builtin_bit_cast(uint32_t, v);
}

template <bool CLAMPED, bool SMALL>  // SMALL: a tile of few rows or few columns (mok::tile_placement), else a full tile
__device__ __forceinline__ void forward(const MokActResidue& p, const MokActTask& t, const AccFrag& acc, const MokCounters& counters) {
  const int tid = fresh_tid();
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int half = lane >> 5;
  unsigned char* stage = pipelink_smem + pipelink_mok_act_arena();
  // One pair of fragments -- gate values and up values of the same 32 routed rows x 32 columns -> 32 x 32 codes and
  // 32 scale bytes in the LDS tile; trow = the lane's tile-local routed row, tcol = the block's tile-local first column.
  auto requantise = [&](const v16f& gate, const v16f& up, int trow, int tcol) {
    float h[16];
    float amax = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; r += 2) {
      h[r] = swiglu<CLAMPED>(gate[r], up[r], p.swiglu_limit);
      h[r + 1] = swiglu<CLAMPED>(gate[r + 1], up[r + 1], p.swiglu_limit);
      amax = fmaxf(fmaxf(amax, fabsf(h[r])), fabsf(h[r + 1]));
    }
    // the other 16 columns of this row's block live in lane ^ 32
    amax = fmaxf(amax, __shfl_xor(amax, 32));
    // The block's scale comes from the largest bf16-rounded magnitude; rounding is monotonic,
    // so that is the rounded largest magnitude.
    const f32x2 am = {amax, 0.0f};
    const uint32_t am_bits = __builtin_bit_cast(uint32_t, __builtin_convertvector(am, bf16x2));
    int e = (int)((am_bits >> 7) & 0xFFu) - 8;  // floor(log2(amax)) - 8 + 127
    e = e < 0 ? 0 : e;                          // amax < 2^-118: scale byte 0
    // 2^(e - 127), a denormal for byte 0; the conversion only looks at the exponent the byte stands for
    const uint32_t scale_bits = (uint32_t)e << 23;
    const float scale = __uint_as_float(scale_bits > 0x00400000u ? scale_bits : 0x00400000u);
    const float limit = __uint_as_float(((uint32_t)(e + 8) << 23) | 0x00600000u);  // 448 * 2^(e - 127), e <= 246
    unsigned char* dst = stage + trow * STAGE_PITCH + tcol + 4 * half;
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<uint32_t*>(dst + 8 * q) = quantise4(h[4 * q], h[4 * q + 1], h[4 * q + 2], h[4 * q + 3], limit, scale);
    if (half == 0) stage[STAGE_SCALE_OFF + trow * 4 + (tcol >> 5)] = (uint8_t)e;
  };
  // ---- activation + requant into an LDS tile [256 rows][128 codes] + [256 rows][4 scales] ----
  const int placement = tile_placement(t.row_end - t.row_begin, p.cols - t.col_begin);
  if constexpr (!SMALL) {
    (void)placement;
    // (a wave whose rows or columns all lie past the end computes on an accumulator the GEMM owner
    // cleared and did not fill; a branch around the arithmetic for it costs every wave spills)
#pragma unroll
    for (int a = 0; a < 2; ++a) {  // gate fragments a, up fragments a + 2: same rows, same columns
#pragma unroll
      for (int b = 0; b < XFRAGS; ++b)
        requantise(from_acc(acc.v[a][b]), from_acc(acc.v[a + 2][b]), xrow0(wave, b) + (lane & 31), wrow0(wave, a));
    }
  } else {
    // a tile of few rows or few columns: 64 routed rows per wave, one or two pairs of fragments (mok::SmallPlacement)
    const SmallPlacement sp = small_placement(placement, __builtin_amdgcn_readfirstlane(wave));
#pragma unroll
    for (int b = 0; b < 2; ++b) requantise(from_acc(acc.v[0][b]), from_acc(acc.v[2][b]), sp.xr0 + 32 * b + (lane & 31), sp.wr[0]);
    if (placement == TILE_SMALL_COLS) {
#pragma unroll
      for (int b = 0; b < 2; ++b) requantise(from_acc(acc.v[1][b]), from_acc(acc.v[3][b]), sp.xr0 + 32 * b + (lane & 31), sp.wr[1]);
    }
  }
  __syncthreads();
  // ---- coalesced write-out: a row is 128 bytes = 8 lanes x 16 bytes, 8 rows per wave store ----
  // Stores of `hidden` are device-scope (cache policy bit 4, sc1): they go through to memory, where a workgroup on
  // another XCD -- a down tile of the same launch, once the row tile's counter says so -- reads them.
  const int chunk = lane & 7;
  const bool col_ok = t.col_begin + chunk * 16 < p.cols;  // column extents are multiples of 32
  const __amdgpu_buffer_rsrc_t out_q =
      __builtin_amdgcn_make_buffer_rsrc(p.hidden_q, 0, (int)((uint32_t)p.rows * (uint32_t)p.ld_q), 0x00020000);
#pragma unroll
  for (int it = 0; it < TILE_X / (THREADS / 64) / 8; ++it) {
    const int trow = wave * (TILE_X / (THREADS / 64)) + it * 8 + (lane >> 3);
    const int row = t.row_begin + trow;
    if (row < t.row_end && col_ok) {
      const v4i v = *reinterpret_cast<const v4i*>(stage + trow * STAGE_PITCH + chunk * 16);
      __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), out_q,
                                             (int)((uint32_t)row * (uint32_t)p.ld_q + (uint32_t)(t.col_begin + chunk * 16)), 0, 16);
    }
  }
  static_assert(THREADS == TILE_X, "one thread per routed row writes the row's scale bytes");
  {
    const int row = t.row_begin + tid;
    if (row < t.row_end) {
      const uint32_t sc = *reinterpret_cast<const uint32_t*>(stage + STAGE_SCALE_OFF + tid * 4);
      uint8_t* out = p.hidden_sc + (int64_t)row * p.ld_sc + (t.col_begin >> 5);
      if (t.col_begin + TILE_W / 2 <= p.cols) {
        // col_begin is a multiple of 128: dword aligned
        __hip_atomic_store(reinterpret_cast<uint32_t*>(out), sc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      } else {
        for (int j = 0; t.col_begin + 32 * j < p.cols; ++j)
          __hip_atomic_store(out + j, (uint8_t)(sc >> (8 * j)), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  // The tile is counted when all of it is in memory: every wave waits until its own stores above have been written
  // through (a store leaves the wave's vector-memory count when it is acknowledged; the barrier's workgroup-scope
  // fence does not wait for that), then the workgroup meets, then one thread counts the tile.  The row tile's counter
  // reaches the number of gate/up column tiles when all of its `hidden` can be read by any workgroup
  // (campaigns/mok/port/framework/interp_fwd.cu:174-213: the reference's act -> down dependency).
  if (t.counter_idx >= 0 && counters.base) __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0)
  __syncthreads();  // also: the staging tile shares LDS with the GEMM ring of the next tile
  if (t.counter_idx >= 0 && counters.base && tid == 0)
    __hip_atomic_fetch_add(counters.base + t.counter_idx, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace mok_act_owner

extern "C" __device__ void mok_act_init(const void* view) { (void)view; }

extern "C" __device__ void mok_act_fwd(const void* view, const MokActTask* task, const MokCounters* counters,
                                       uint32_t* phase, const mok::AccFrag* acc) {
  (void)phase;
  const auto& p = *static_cast<const MokActResidue*>(static_cast<const pipelink_host_view*>(view)->residue);
  if (pipelink_mok_clamp())
    mok_act_owner::forward<true, false>(p, *task, *acc, *counters);
  else
    mok_act_owner::forward<false, false>(p, *task, *acc, *counters);
}

// The same for a tile whose accumulator is in the small placement (mok::tile_placement of the task's extent is not
// TILE_FULL): the caller tells the two apart, as it does for the GEMM owner's exports.
extern "C" __device__ void mok_act_fwd_small(const void* view, const MokActTask* task, const MokCounters* counters,
                                             uint32_t* phase, const mok::AccFrag* acc) {
  (void)phase;
  const auto& p = *static_cast<const MokActResidue*>(static_cast<const pipelink_host_view*>(view)->residue);
  if (pipelink_mok_clamp())
    mok_act_owner::forward<true, true>(p, *task, *acc, *counters);
  else
    mok_act_owner::forward<false, true>(p, *task, *acc, *counters);
}
#else  // PIPELINK_EMIT: host-evaluated annotations only
#include "../include/mok_abi.h"
#endif

PL_STAGE("mok.act", "0.1.0-gptoss");
PL_PARAMS(MokActResidue);
PL_TOPOLOGY(true, "static");
// clamp on/off is a link-time variant (campaigns/mok/port/act_gptoss/act.cu:246-249)
PL_VARIANT(0, {{"pipelink_mok_clamp", 0}});
PL_VARIANT(1, {{"pipelink_mok_clamp", 1}});
PL_EXPORT(mok_act_init, mok_act_init, "extern \"C\" __device__ void mok_act_init(const void* view);");
PL_EXPORT(mok_act_fwd, mok_act_fwd,
          "extern \"C\" __device__ void mok_act_fwd(const void* view, const MokActTask* task, "
          "const MokCounters* counters, uint32_t* phase, const mok::AccFrag* acc);");
PL_EXPORT(mok_act_fwd_small, mok_act_fwd_small,
          "extern \"C\" __device__ void mok_act_fwd_small(const void* view, const MokActTask* task, "
          "const MokCounters* counters, uint32_t* phase, const mok::AccFrag* acc);");
PL_SERVE(act_init, "mok_act_init");
PL_SERVE(act_fwd, "mok_act_fwd");
PL_SERVE(act_fwd_small, "mok_act_fwd_small");
// staging tile for the coalesced write-out; lives while no GEMM ring slot is in use
PL_CLAIM("pipelink_mok_act_arena", "smem", 256 * 144 + 256 * 4, 1024, "phase:instr_act");
// host contract (campaigns/mok/port/act/act.cu:280-330 in the reference)
PL_HOST_GROUP("mok.act.params", "mok_act");
PL_HOST_ABI_TYPE(2, MokActResidue);
MOK_HOST_SCALARS();
PL_HOST_CHANNEL(1, "hidden_q", 8, "write", "mok.routed_rows, mok.ld_q_i", false);
PL_HOST_CHANNEL(2, "hidden_sc", 8, "write", "mok.routed_rows, mok.ld_sc_i", false);
PL_USES("pipelink_mok_clamp");
PL_USES("pipelink_mok_act_arena");
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
