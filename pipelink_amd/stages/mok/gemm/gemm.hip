// Owner package mok.gemm: MXFP8 grouped-GEMM mainloop for one workgroup tile on gfx950.
//
// Replaces the reference's routed forward ops of campaigns/mok/port/gemm/gemm.cu:150-162
// (expert_grouped_gemm_kernel<false>, body in the absent mixture-of-kittens submodule):
//   gate|up[r, n] = sum_k deq(x[row_token[r], k]) * deq(W[e][n, k])      (fp32 accumulate)
//   y[r, n]       = sum_k deq(hidden[r, k])      * deq(Wd[e][n, k])      -> bf16
// Operand roles are swapped with respect to the usual "A = activations": the weight rows
// feed the MFMA A operand and the routed rows the B operand, so one lane ends up holding
// four consecutive output columns of one routed row, which is what the requantising
// epilogue and the bf16 store want.
//
// LDS: two rings of 16 KB buffers, one for the routed rows and one for the weight rows.  A
// buffer holds 64 contraction bytes -- one MFMA step, "slot" below -- of 256 rows, row-major.
// One buffer_load_dwordx4 ... lds moves 16 rows: four lanes cover the 64 contiguous bytes of a
// row.  The four 16-byte chunks of a row are stored at position chunk ^ ((row / 4) % 4), which
// makes a fragment read (16 lanes = 16 consecutive rows, one chunk each) touch 16 different
// 16-byte bank groups.  The weight ring has `depth` buffers (a link-time handle) and takes
// one slot per step; weight codes are stored K-tiled in HBM ([K/64][rows][64 bytes]), so the
// 16 rows of a load are 1 KB of contiguous memory.  The routed-row ring has depth + 1 buffers and takes two slots -- the
// two halves of one 128-byte line per row -- every second step, the two loads of a row back
// to back: issued like that the pair costs the memory system what one full-line request
// costs, issued a step apart it costs about a fifth more time (measured).  Behind the rings:
// four 1 KB buffers of weight block scales (stored slot-major in HBM, one dword = 128
// contraction bytes per row, so a tile's share is one contiguous load every second slot) and
// two 4 KB buffers of routed-row scales (row-major in HBM because rows are gathered; 16 bytes
// per row = eight slots' worth, fetched every eighth slot while the previous eight are in use).
//
// Schedule: one wave per SIMD, 128 x 128 outputs per wave in 256 accumulator registers.
// While the 16 MFMAs of slot j run, the wave reads the operands of slot j+1 from LDS into a
// second register set and the loads of the following slots are in flight, so neither the LDS
// latency nor the L2 latency sits between two MFMAs.  One s_barrier per slot; it only waits
// for what was issued `depth` - 1 steps earlier.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <type_traits>
#include <utility>
#include "../include/mok_device.hpp"

extern "C" __device__ int pipelink_mok_gemm_depth();  // ring slots (2 or 4), bound at link time
#include "load_counts.hpp"

extern "C" __device__ int pipelink_mok_gemm_head();   // byte offset of the rings' first two buffers + scale buffers in dynamic LDS
extern "C" __device__ int pipelink_mok_gemm_arena();  // byte offset of the rings' other buffers

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mok_gemm_owner {
using namespace mok;

constexpr int WAVES = THREADS / 64;
constexpr int X_GROUPS = TILE_X / 16 / WAVES;  // 16-row load groups per wave (4)
constexpr int W_GROUPS = TILE_W / 16 / WAVES;  // (4)
constexpr int X_LOADS = 2 * X_GROUPS;          // loads of one routed-row pair issue (even steps)
constexpr int W_LOADS = W_GROUPS;              // loads of one weight slot issue (every step)

// Loads are buffer loads: a 128-bit resource (base address and byte extent, in scalar
// registers), a 32-bit lane offset that is fixed for the tile, and the contraction offset as
// the instruction's scalar offset -- no address arithmetic per load, and a read past the
// extent returns zeros instead of faulting.  One operand of one expert is 16 MiB below 4 GiB
// (the host checks).
typedef __amdgpu_buffer_rsrc_t rsrc_t;

// Lane offset of the rows and columns a tile has past the end of its expert's rows or of the
// weight matrix: beyond every extent (the host keeps operands 16 MiB below 4 GiB), so the
// load brings zeros without touching memory, and the matrix pipe multiplies zeros there,
// which costs it far less power than multiplying a copy of the last row would.  Nothing
// depends on the zeros: those outputs are never stored.
constexpr uint32_t PAST_THE_END = 0xFF000000u;

__device__ __forceinline__ rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);  // raw, 32-bit data
}
// 16 (4) bytes per lane, buffer -> LDS; lane i lands at lds + 16*i (4*i)
__device__ __forceinline__ void buf16_to_lds(rsrc_t r, uint32_t lane_off, uint32_t uni_off, unsigned char* lds) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lptr_t)lds, 16, (int)lane_off, (int)uni_off, 0, 0);
}
__device__ __forceinline__ void buf4_to_lds(rsrc_t r, uint32_t lane_off, uint32_t uni_off, unsigned char* lds) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lptr_t)lds, 4, (int)lane_off, (int)uni_off, 0, 0);
}
// The same at device scope (cache policy bit 4, sc1): the load does not trust a line that another XCD's workgroup may
// have written during this launch.  Used for what one workgroup of the launch writes and another reads where a cache
// line can hold both finished and unfinished parts: the scale rows of `hidden` (a line spans rows of different row
// tiles) and the readiness counters.
__device__ __forceinline__ void buf16_to_lds_device_scope(rsrc_t r, uint32_t lane_off, uint32_t uni_off, unsigned char* lds) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lptr_t)lds, 16, (int)lane_off, (int)uni_off, 0, 16);
}
__device__ __forceinline__ void buf4_to_lds_device_scope(rsrc_t r, uint32_t lane_off, uint32_t uni_off, unsigned char* lds) {
  __builtin_amdgcn_raw_ptr_buffer_load_lds(r, (lptr_t)lds, 4, (int)lane_off, (int)uni_off, 0, 16);
}

struct Loader {
  rsrc_t x;                       // activations (all rows)
  rsrc_t w;                       // this expert's weight matrix (gate or up or down, by wave)
  rsrc_t xsc;                     // routed rows' scales, row-major
  rsrc_t wsc;                     // this expert's weight scales (gate or up or down, by wave), slot-major
  uint32_t wsc_pair_pitch;        // bytes between two 128-byte pairs of the weight scales
  uint32_t w_slot_pitch;          // bytes between two 64-byte slots of the weight codes (K-tiled: rows x 64)
  uint32_t wscsrc;                // this thread's weight row: its dword of block scales
  uint32_t xscsrc;                // this thread's routed row in the scale matrix
  uint32_t xsrc[X_GROUPS];        // this lane's 16 bytes of its row in each group, at k = 0
  uint32_t wsrc[W_GROUPS];
  int dst;                        // buffer-relative LDS byte offset of the wave's first group (both rings)
};

// LDS areas of one workgroup.  The first two buffers of each ring and the scale buffers (the
// "head", claimed for the whole kernel) take the next tile's first loads while the current
// tile's epilogue runs; the other buffers (the "arena", claimed for the GEMM phase only) share
// their LDS with the epilogue's staging tile.
//   head : X0 X1 W0 W1 | 4 x 1 KB weight scales | 2 x 4 KB routed-row scales | staged task: 1 KB row tokens, 256 B counter
//   arena: X2 .. X[DEPTH] | W2 .. W[DEPTH-1]
constexpr int STAGED_TOKEN_BYTES = TILE_X * 4;  // row_token of the staged tile's rows
constexpr int STAGED_PEEK_BYTES = 256;          // one wave's copies of the readiness counter it depends on
constexpr int HEAD_BYTES = 4 * BUF_BYTES + WSCALE_BYTES + XSCALE_BYTES + STAGED_TOKEN_BYTES + STAGED_PEEK_BYTES;
template <int DEPTH>
struct Rings {
  unsigned char* head;
  unsigned char* arena;
  __device__ __forceinline__ Rings()
      : head(pipelink_smem + pipelink_mok_gemm_head()), arena(pipelink_smem + pipelink_mok_gemm_arena()) {}
  __device__ __forceinline__ unsigned char* x(int b) const {  // routed-row buffer b of DEPTH + 1
    return b < 2 ? head + b * BUF_BYTES : arena + (b - 2) * BUF_BYTES;
  }
  __device__ __forceinline__ unsigned char* w(int b) const {  // weight buffer b of DEPTH
    return b < 2 ? head + (2 + b) * BUF_BYTES : arena + (DEPTH - 1 + b - 2) * BUF_BYTES;
  }
  __device__ __forceinline__ unsigned char* wscale() const { return head + 4 * BUF_BYTES; }
  __device__ __forceinline__ unsigned char* xscale() const { return head + 4 * BUF_BYTES + WSCALE_BYTES; }
  __device__ __forceinline__ unsigned char* tokens() const { return head + 4 * BUF_BYTES + WSCALE_BYTES + XSCALE_BYTES; }
  __device__ __forceinline__ unsigned char* peek() const { return tokens() + STAGED_TOKEN_BYTES; }
};

__device__ __forceinline__ int swizzle(int row) { return (row >> 2) & 3; }

// A wave whose whole 128 x 128 share of the tile lies past the end of the expert's rows, or past
// the last output column, has nothing to multiply: it keeps loading its share of the tile's
// operands for the other waves and meets every barrier, and leaves the matrix pipe and its
// operand reads alone (the accumulator it hands on is never looked at: its outputs are not
// stored).  `cols` is the number of output columns (weight rows of one matrix).
__device__ __forceinline__ bool wave_idle(const MokGemmTask& t, int cols) {
  const int wave = __builtin_amdgcn_readfirstlane(fresh_tid() >> 6);
  const bool no_rows = t.row_begin + xrow0(wave, 0) >= t.row_end;
  const bool no_cols = t.col_begin + wave_w(wave) * 64 >= cols;  // the wave's lowest column, both ops
  return no_rows || no_cols;
}

// Issue the weight rows of slot j into weight buffer `buf`, preceded by the scale loads that
// go with slot j.  Scale loads go first so that they are older than tile loads of the same
// step: the outstanding-load counts the waits use only count tile loads, which errs on the
// side of waiting for more.  J8 is j % 8 where the caller knows it at compile time, else -1.
template <int J8 = -1, int DEPTH>
__device__ __forceinline__ void issue_w(const Loader& ld, const Rings<DEPTH>& r, int j, int buf) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t kbyte = (uint32_t)j * K_SLOT;
  const int j8 = J8 >= 0 ? J8 : (j & 7);
  // every eighth slot: 16 scale bytes of each routed row (this slot and the next seven)
  if (j8 == 0) buf16_to_lds_device_scope(ld.xsc, ld.xscsrc, kbyte >> 5, r.xscale() + ((j >> 3) & 1) * (TILE_X * 16) + wave * 1024);
  // every second slot: the tile's weight scales of this pair, one row per thread
  if ((j8 & 1) == 0)
    buf4_to_lds(ld.wsc, ld.wscsrc, (uint32_t)(j >> 1) * ld.wsc_pair_pitch, r.wscale() + (j8 >> 1) * (TILE_W * 4) + wave * 256);
  unsigned char* dst = r.w(buf) + ld.dst;
  const uint32_t wslot = (uint32_t)j * ld.w_slot_pitch;
#pragma unroll
  for (int i = 0; i < W_GROUPS; ++i) buf16_to_lds(ld.w, ld.wsrc[i], wslot, dst + i * 1024);
}

// Issue row groups G0 .. G1-1 of the routed rows of slots j and j+1 (j even: the two halves of a
// 128-byte line) into routed-row buffers buf0 and buf1, the two loads of a row group back to back.
template <int G0, int G1, int DEPTH>
__device__ __forceinline__ void issue_x_groups(const Loader& ld, const Rings<DEPTH>& r, int j, int buf0, int buf1) {
  const uint32_t kbyte = (uint32_t)j * K_SLOT;
  unsigned char* dst0 = r.x(buf0) + ld.dst;
  unsigned char* dst1 = r.x(buf1) + ld.dst;
#pragma unroll
  for (int i = G0; i < G1; ++i) {
    buf16_to_lds(ld.x, ld.xsrc[i], kbyte, dst0 + i * 1024);
    buf16_to_lds(ld.x, ld.xsrc[i], kbyte + K_SLOT, dst1 + i * 1024);
  }
}

// The same loads one at a time, for the steady-state steps that place every load between two
// particular MFMAs.  Load L of the step that issues weight slot j (J8 = j % 8); the routed rows
// belong to the pair of slots that starts at j (even step) or at j - 1 (odd step) and go into
// routed-row buffers xb0 / xb1:
//   even step: 0 routed-row scales (if J8 == 0), 1 weight scales, 2..5 routed rows (group (L-2)/2,
//              half (L-2)%2), 6..9 weight rows
//   odd step:  0..3 routed rows (group 2 + L/2, half L%2), 4..7 weight rows
template <bool ODD, int J8, int L, int DEPTH>
__device__ __forceinline__ void issue_one(const Loader& ld, const Rings<DEPTH>& r, int j, int wbuf, int xb0, int xb1) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t kbyte = (uint32_t)j * K_SLOT;
  constexpr int XL = ODD ? L : L - 2;       // routed-row load 0..3 of this step
  constexpr int WL = ODD ? L - 4 : L - 6;   // weight group
  if constexpr (!ODD && L == 0) {
    if constexpr (J8 == 0) buf16_to_lds_device_scope(ld.xsc, ld.xscsrc, kbyte >> 5, r.xscale() + ((j >> 3) & 1) * (TILE_X * 16) + wave * 1024);
  } else if constexpr (!ODD && L == 1) {
    static_assert(ODD || (J8 & 1) == 0, "even steps issue even slots");
    buf4_to_lds(ld.wsc, ld.wscsrc, (uint32_t)(j >> 1) * ld.wsc_pair_pitch, r.wscale() + (J8 >> 1) * (TILE_W * 4) + wave * 256);
  } else if constexpr (XL >= 0 && XL < 4) {
    constexpr int G = (ODD ? 2 : 0) + XL / 2, H = XL % 2;
    const uint32_t kpair = ODD ? kbyte - K_SLOT : kbyte;  // the pair's first slot
    buf16_to_lds(ld.x, ld.xsrc[G], kpair + H * K_SLOT, r.x(H ? xb1 : xb0) + ld.dst + G * 1024);
  } else if constexpr (WL >= 0 && WL < W_GROUPS) {
    buf16_to_lds(ld.w, ld.wsrc[WL], (uint32_t)j * ld.w_slot_pitch, r.w(wbuf) + ld.dst + WL * 1024);
  }
}

// MFMA 32x32x64 f8f6f4 operand of lane (row = lane % 32, half = lane / 32): registers 0-3
// hold 16 bytes of the step's first 32-element block, registers 4-7 16 bytes of its second
// block; the scale of block 0 is taken from lanes 0-31 and that of block 1 from lanes 32-63
// (measured on gfx950 with a one-instruction probe).  So a lane reads chunks half and
// half + 2 of its row; with the XOR swizzle the second is the first with bit 5 flipped.
__device__ __forceinline__ v8i read_frag(const unsigned char* slot, int off) {
  const v4i lo = *reinterpret_cast<const v4i*>(slot + off);
  const v4i hi = *reinterpret_cast<const v4i*>(slot + (off ^ 32));
  v8i r;
  r.s0 = lo.x; r.s1 = lo.y; r.s2 = lo.z; r.s3 = lo.w;
  r.s4 = hi.x; r.s5 = hi.y; r.s6 = hi.z; r.s7 = hi.w;
  return r;
}

// A zeroed accumulator fragment.  Written by one instruction of the matrix pipe (an integer MFMA of zeros, eight
// passes) instead of sixteen register writes: a wave issues in order, one instruction every four or five clocks, and 256
// writes per tile are half a microsecond in which it issues nothing else.  (The zero is opaque to the compiler, which
// would otherwise fold the product back into the writes.)
// The instruction is written out so that its result is born in the accumulator registers (left to the compiler it
// may be born in vector registers and copied, which the mainloop has none to spare for); nothing reads the fragment
// for hundreds of instructions, so the matrix pipe's result latency needs no attention here.
__device__ __forceinline__ v16f zero_fragment() {
  long z = 0;
  v16f f;
  asm volatile("v_mfma_i32_32x32x16_i8 %0, %1, %1, 0" : "=a"(f) : "v"(z));
  return f;
}

// Workgroup barrier without the release/acquire fence of __syncthreads(): a fence would
// drain every outstanding global->LDS load (vmcnt(0)) and serialise the ring.  Ordering of
// the LDS traffic is by the explicit s_waitcnt in front of it.
__device__ __forceinline__ void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

// wait until at most N global loads are outstanding and every LDS read has returned
template <int N>
__device__ __forceinline__ void wait_loads_and_reads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 0xF) | ((N >> 4) << 14));
}

struct Operands {
  v8i x[XFRAGS], w[WFRAGS];
};

__device__ __forceinline__ void read_operands(Operands& o, const unsigned char* xbuf, const unsigned char* wbuf,
                                              const int (&xoff)[XFRAGS], const int (&woff)[WFRAGS]) {
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) o.x[b] = read_frag(xbuf, xoff[b]);
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) o.w[a] = read_frag(wbuf, woff[a]);
}

// s_waitcnt needs an immediate: the few counts the last steps of a tile can ask for
__device__ __forceinline__ void wait_loads_and_reads_dyn(int n) {
  switch (n) {
    case 0: wait_loads_and_reads<0>(); break;
    case 4: wait_loads_and_reads<4>(); break;
    case 8: wait_loads_and_reads<8>(); break;
    case 12: wait_loads_and_reads<12>(); break;
    case 16: wait_loads_and_reads<16>(); break;
    case 20: wait_loads_and_reads<20>(); break;
    case 24: wait_loads_and_reads<24>(); break;
    default: wait_loads_and_reads<0>(); break;  // waiting for everything is always right
  }
}

// Block scales of the 128-byte pair that starts at slot j (j even): one dword per row; lanes
// of the upper half use blocks 1 and 3, shifted down into bytes 0 and 2 where the MFMA's
// op_sel picks them (0 in the pair's first slot, 2 in its second).  The routed rows' dwords
// sit 16 bytes apart (a 4-way bank conflict on four small reads per pair).
template <int J8 = -1, bool SHIFT = true>
__device__ __forceinline__ void read_scales(int (&sx)[XFRAGS], int (&sw)[WFRAGS], const unsigned char* wscale,
                                            const unsigned char* xscale, int j, const int (&xscoff)[XFRAGS],
                                            const int (&wscoff)[WFRAGS], int half) {
  const int c = (J8 >= 0 ? J8 : (j & 7)) >> 1;
  const unsigned char* xbuf = xscale + ((j >> 3) & 1) * (TILE_X * 16);
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) {
    const uint32_t v = *reinterpret_cast<const uint32_t*>(xbuf + 4 * c + xscoff[b]);
    sx[b] = (int)(SHIFT ? v >> (8 * half) : v);
  }
  const unsigned char* wbuf = wscale + c * (TILE_W * 4);
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) {
    const uint32_t v = *reinterpret_cast<const uint32_t*>(wbuf + wscoff[a]);
    sw[a] = (int)(SHIFT ? v >> (8 * half) : v);
  }
}
// second half of read_scales<.., false>
__device__ __forceinline__ void shift_scales(int (&sx)[XFRAGS], int (&sw)[WFRAGS], int half) {
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) sx[b] = (int)((uint32_t)sx[b] >> (8 * half));
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) sw[a] = (int)((uint32_t)sw[a] >> (8 * half));
}

template <bool ODD>
__device__ __forceinline__ void mma_step(const Operands& o, const int (&sx)[XFRAGS], const int (&sw)[WFRAGS],
                                         AccFrag& acc) {
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a)
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b)
      acc.v[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(o.w[a], o.x[b], acc.v[a][b], 0, 0, ODD ? 2 : 0,
                                                                    sw[a], ODD ? 2 : 0, sx[b]);
}

// Looking ahead.  While a tile is multiplied the framework names the task that comes after it; `stage` asks memory
// for what that task's prefetch will want first and would otherwise wait for: the row_token entries of its rows
// (gate/up op) and the readiness counter its rows depend on (down op in a launch of both GEMMs), both straight into
// LDS.  The loads are younger than everything the running mainloop waits for and have landed when it ends.
__device__ __forceinline__ bool waits(const MokGemmTask& t, const MokCounters& counters) {
  return t.wait_target > 0 && t.counter_idx >= 0 && counters.base != nullptr;
}
__device__ __forceinline__ void stage(const MokGemmResidue& g, const MokGemmTask& t, const MokCounters& counters) {
  const int tid = fresh_tid();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const Rings<2> r;  // the staged areas do not depend on the depth
  if (t.op == MOK_GEMM_FWD_ROUTED_GATE_UP && g.row_token) {
    const int row = t.row_begin + tid;
    const rsrc_t tok = make_rsrc(g.row_token, (uint32_t)g.hidden.rows * 4u);  // one entry per routed row
    buf4_to_lds(tok, row < t.row_end ? (uint32_t)row * 4u : PAST_THE_END, 0, r.tokens() + wave * 256);
  }
  if (waits(t, counters) && wave == 0) {
    const rsrc_t cnt = make_rsrc(counters.base, (uint32_t)(t.counter_idx + 1) * 4u);
    buf4_to_lds_device_scope(cnt, (uint32_t)t.counter_idx * 4u, 0, r.peek());  // 64 copies of one word
    (void)lane;
  }
}
// what `stage` saw of the task's counter: true if the rows the task reads were complete then (or it depends on none)
__device__ __forceinline__ bool staged_ready(const MokGemmTask& t, const MokCounters& counters) {
  if (!waits(t, counters)) return true;
  const Rings<2> r;
  return *reinterpret_cast<const volatile int32_t*>(r.peek()) >= t.wait_target;
}
// Waits until the rows the task reads are complete: one thread polls the counter at device scope, the others wait at
// the barrier.  A bounded poll: after WAIT_POLLS probes (a few tens of milliseconds; a wait that can be met takes
// microseconds) it raises the launch's status word and goes on (the tile then multiplies whatever `hidden` holds), so a
// launch never spins for ever.  The first wait that gives up also says so in a word of the launch's own, which every
// waiting thread looks at before it polls and every 256 polls: the launch's results are void by then, and its other
// waits end at once instead of each running to the limit.
constexpr uint32_t WAIT_POLLS = 1u << 14;
__device__ __forceinline__ void wait_rows(const MokGemmTask& t, const MokCounters& counters) {
  if (!waits(t, counters)) return;
  if (threadIdx.x == 0) {
    uint32_t* const gave_up = counters.status ? counters.status + (MOK_WS_GAVE_UP - MOK_WS_STATUS) : nullptr;
    uint32_t limit = WAIT_POLLS;
    if (counters.status) {  // the host may shorten the wait (MOK_WS_POLL_LIMIT)
      const uint32_t asked = __hip_atomic_load(counters.status + (MOK_WS_POLL_LIMIT - MOK_WS_STATUS), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (asked != 0) limit = asked;
    }
    bool ok = false;
    for (uint32_t spin = 0;; ++spin) {
      ok = __hip_atomic_load(counters.base + t.counter_idx, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >= t.wait_target;
      if (ok || spin >= limit) break;
      if ((spin & 255u) == 0 && gave_up && __hip_atomic_load(gave_up, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) != 0) break;
      __builtin_amdgcn_s_sleep(8);
    }
    if (!ok && counters.status) {
      __hip_atomic_fetch_or(counters.status, (uint32_t)MOK_STATUS_WAIT_GAVE_UP, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(gave_up, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  __syncthreads();
}

// The two operands of a task as this wave sees them.
struct Views {
  const MokMxView& act;  // routed rows: x (gate/up op) or hidden (down op)
  const MokMxView& w;    // weight rows this wave loads: gate or up (by wave) or down
};
__device__ __forceinline__ Views views_of(const MokGemmResidue& g, const MokGemmTask& t) {
  const int wave = __builtin_amdgcn_readfirstlane(fresh_tid() >> 6);
  const bool gate_up = t.op == MOK_GEMM_FWD_ROUTED_GATE_UP;
  const MokMxView* a = gate_up ? &g.x : &g.hidden;
  const MokMxView* w = gate_up ? (wave < WAVES / 2 ? &g.w_gate : &g.w_up) : &g.w_down;
  return Views{*a, *w};
}

// The gathered part of a tile's loader: routed row -> source row goes through row_token for the gate/up op, a
// dependent load, which `stage` has taken ahead: the tokens are read from LDS (those of rows past the end are zero there).
// (`few`: a tile of at most 64 rows in the deep ring below, whose wave w loads routed rows 16 w .. 16 w + 15: xsrc[0] only.)
__device__ __forceinline__ void gather_rows(const MokGemmResidue& g, const Views& v, const MokGemmTask& t, GemmCarry& c, bool few = false) {
  const int tid = fresh_tid();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const bool gate_up = t.op == MOK_GEMM_FWD_ROUTED_GATE_UP;
  const MokMxView& act = v.act;
  const bool gathered = gate_up && g.row_token;
  const int32_t* staged_token = reinterpret_cast<const int32_t*>(Rings<2>().tokens());
  const int lrow = lane >> 2;
  const int chunk = 16 * ((lane & 3) ^ swizzle(lrow));
#pragma unroll
  for (int i = 0; i < X_GROUPS; ++i) {
    const int trow = few ? wave * 16 + lrow : (wave * X_GROUPS + i) * 16 + lrow;  // tile-local routed row
    const int row = t.row_begin + trow;
    const int safe = row < t.row_end ? row : t.row_end - 1;
    const int src = gathered ? staged_token[trow] : safe;
    c.xsrc[i] = row < t.row_end ? (uint32_t)src * (uint32_t)act.ld_q + chunk : PAST_THE_END;
  }
  // routed-row scales: thread tid fetches row tid's 16-byte piece
  const int row = t.row_begin + tid;
  const int safe = row < t.row_end ? row : t.row_end - 1;
  const int src = gathered ? staged_token[tid] : safe;
  c.xscsrc = row < t.row_end ? (uint32_t)src * (uint32_t)act.ld_sc : PAST_THE_END;
}

// Loader of a tile: lane -> (row lane/4 of a 16-row group, LDS position lane%4); it fetches the
// chunk that belongs at that position.  Groups start at multiples of 16 rows, so the swizzle
// of a row only depends on its place in the group.
__device__ __forceinline__ Loader make_loader(const Views& v, const MokGemmTask& t, const GemmCarry& c) {
  const int tid = fresh_tid();
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: resources chosen by it stay scalar
  const bool gate_up = t.op == MOK_GEMM_FWD_ROUTED_GATE_UP;
  const int expert = __builtin_amdgcn_readfirstlane(t.expert);
  const MokMxView& act = v.act;
  Loader ld;
  const int lrow = lane >> 2;
  const int chunk = 16 * ((lane & 3) ^ swizzle(lrow));
#pragma unroll
  for (int i = 0; i < X_GROUPS; ++i) ld.xsrc[i] = c.xsrc[i];
  ld.xscsrc = c.xscsrc;
  ld.x = make_rsrc(act.q, (uint32_t)act.rows * (uint32_t)act.ld_q);
  ld.xsc = make_rsrc(act.sc, (uint32_t)act.rows * (uint32_t)act.ld_sc);
  ld.dst = wave * X_GROUPS * 1024;
  static_assert(X_GROUPS == W_GROUPS, "one wave offset serves both rings");
  const MokMxView& wv = v.w;
#pragma unroll
  for (int i = 0; i < W_GROUPS; ++i) {
    const int wl = (wave * W_GROUPS + i) * 16 + lrow;  // tile-local weight row
    const int col = t.col_begin + (gate_up ? (wl & (TILE_W / 2 - 1)) : wl);
    ld.wsrc[i] = col < wv.rows ? (uint32_t)col * (uint32_t)K_SLOT + chunk : PAST_THE_END;  // weights are K-tiled: [K/64][rows][64]
  }
  ld.w = make_rsrc(wv.q + (int64_t)expert * wv.expert_pitch_q, (uint32_t)wv.rows * (uint32_t)wv.k);
  ld.w_slot_pitch = (uint32_t)wv.rows * (uint32_t)K_SLOT;
  // weight scales, slot-major [pair][row][4]: thread tid fetches tile row tid's dword
  static_assert(THREADS == TILE_W, "one thread per weight row");
  const int col = t.col_begin + (gate_up ? (tid & (TILE_W / 2 - 1)) : tid);
  ld.wsc = make_rsrc(wv.sc + (int64_t)expert * wv.expert_pitch_sc,
                     (uint32_t)((wv.k + K_PAIR - 1) / K_PAIR) * (uint32_t)wv.rows * 4u);
  ld.wscsrc = col < wv.rows ? (uint32_t)col * 4u : PAST_THE_END;
  ld.wsc_pair_pitch = (uint32_t)wv.rows * 4u;
  return ld;
}

// Loads of schedule step u (u < 0: before a tile's first MFMA), in this order: [scale loads]
// [routed rows] [weight rows of slot u + DEPTH].  With DEPTH >= 4 the routed rows of a pair of
// slots are split over two steps, so that every step issues the same 8 tile loads: groups 0-1
// of the pair that starts at slot u + DEPTH on even u, groups 2-3 of the same pair on the odd
// step after it.  With DEPTH == 2 the whole pair is issued on the even step.  Steps -DEPTH and
// 1 - DEPTH only touch head buffers: `prefetch` issues them, and may run while the previous
// tile's epilogue still uses the arena.
template <int DEPTH>
__device__ __forceinline__ void issue_step(const Loader& ld, const Rings<DEPTH>& r, int u, int n, int xb0, int xb1, int wb) {
  constexpr bool SPLIT = DEPTH >= 4;
  const int s = u + DEPTH;
  const int pair = (u & 1) ? s - 1 : s;
  if (pair < n) {
    if (!SPLIT) {
      if ((u & 1) == 0) issue_x_groups<0, X_GROUPS>(ld, r, pair, xb0, xb1);
    } else if ((u & 1) == 0) {
      issue_x_groups<0, X_GROUPS / 2>(ld, r, pair, xb0, xb1);
    } else {
      issue_x_groups<X_GROUPS / 2, X_GROUPS>(ld, r, pair, xb0, xb1);
    }
  }
  if (s < n) issue_w(ld, r, s, wb);
}
// how many tile loads may be in flight behind a slot: load_counts.hpp
using counts::loads_younger_than_slot;
using counts::few_younger;
static_assert(counts::X_LOADS == X_LOADS && counts::W_LOADS == W_LOADS, "the accounting's loads per step are this loader's");
// ---- tiles of at most 64 routed rows: a deeper ring ---------------------------------------------------------------
// Such a tile has a quarter of a full tile's MFMAs and as many steps: it takes as long as its loads take to arrive,
// and a load that is in flight for three steps' time (the full tile's ring) bounds a step from below by a third of
// the latency of a load.  Its routed rows need 4 KB per slot, not 16: the same LDS holds seven slots of 16 KB of
// weight rows + 4 KB of routed rows, the first three in the head (where the tile before leaves room while its
// epilogue uses the arena), four in the arena.  Wave w loads its 64 weight rows as in the full tile and routed rows
// 16 w .. 16 w + 15; one slot per step, all of it at once (five loads a wave).  Scale buffers and their loads are the
// full tile's.  Needs the arena of ring depth 4.
constexpr int FEW_DEPTH = counts::FEW_DEPTH;
constexpr int FEW_HEAD_SLOTS = 3;
constexpr int FEW_X_BYTES = SMALL_EXTENT * K_SLOT;        // 4 KB
constexpr int FEW_SLOT_BYTES = BUF_BYTES + FEW_X_BYTES;   // weight rows, then routed rows
constexpr int FEW_LOADS = counts::FEW_LOADS;              // tile loads of one slot, per wave
static_assert(FEW_LOADS == W_LOADS + 1, "four groups of weight rows and one of routed rows");
static_assert(FEW_HEAD_SLOTS * FEW_SLOT_BYTES <= 4 * BUF_BYTES, "the first slots fit where the full tile's first buffers are");
struct FewRing {
  unsigned char* head;
  unsigned char* arena;
  __device__ __forceinline__ FewRing() : head(pipelink_smem + pipelink_mok_gemm_head()), arena(pipelink_smem + pipelink_mok_gemm_arena()) {}
  __device__ __forceinline__ unsigned char* slot(int pos) const {  // pos = slot number mod FEW_DEPTH
    return pos < FEW_HEAD_SLOTS ? head + pos * FEW_SLOT_BYTES : arena + (pos - FEW_HEAD_SLOTS) * FEW_SLOT_BYTES;
  }
};
// all loads of slot s, into ring position pos: [scale loads] [routed rows] [weight rows]
__device__ __forceinline__ void issue_few(const Loader& ld, const FewRing& ring, const Rings<4>& r, int s, int pos, int n) {
  if (s >= n) return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t kbyte = (uint32_t)s * K_SLOT;
  const int j8 = s & 7;
  if (j8 == 0) buf16_to_lds_device_scope(ld.xsc, ld.xscsrc, kbyte >> 5, r.xscale() + ((s >> 3) & 1) * (TILE_X * 16) + wave * 1024);
  if ((j8 & 1) == 0) buf4_to_lds(ld.wsc, ld.wscsrc, (uint32_t)(s >> 1) * ld.wsc_pair_pitch, r.wscale() + (j8 >> 1) * (TILE_W * 4) + wave * 256);
  unsigned char* base = ring.slot(pos);
  buf16_to_lds(ld.x, ld.xsrc[0], kbyte, base + BUF_BYTES + wave * 1024);
  const uint32_t wslot = (uint32_t)s * ld.w_slot_pitch;
#pragma unroll
  for (int i = 0; i < W_GROUPS; ++i) buf16_to_lds(ld.w, ld.wsrc[i], wslot, base + ld.dst + i * 1024);
}
__device__ __forceinline__ void wait_few(int loads) {  // a multiple of FEW_LOADS, at most (FEW_DEPTH - 1) of them
  switch (__builtin_amdgcn_readfirstlane(loads) / FEW_LOADS) {
    case 0: wait_loads_and_reads<0>(); break;
    case 1: wait_loads_and_reads<FEW_LOADS>(); break;
    case 2: wait_loads_and_reads<2 * FEW_LOADS>(); break;
    case 3: wait_loads_and_reads<3 * FEW_LOADS>(); break;
    case 4: wait_loads_and_reads<4 * FEW_LOADS>(); break;
    case 5: wait_loads_and_reads<5 * FEW_LOADS>(); break;
    default: wait_loads_and_reads<6 * FEW_LOADS>(); break;
  }
}
// which placement the task's tile has: its routed rows that exist, its output columns that exist
__device__ __forceinline__ int placement_of(const MokGemmResidue& g, const MokGemmTask& t) {
  const int cols = (t.op == MOK_GEMM_FWD_ROUTED_GATE_UP ? g.w_gate.rows : g.w_down.rows) - t.col_begin;
  return tile_placement(t.row_end - t.row_begin, cols);
}

template <int DEPTH>
__device__ __forceinline__ void prefetch(const MokGemmResidue& g, const MokGemmTask& t, GemmCarry& c) {
  const Views v = views_of(g, t);
  const int n = v.act.k / K_SLOT;
  if constexpr (DEPTH >= 4) {
    if (placement_of(g, t) == TILE_SMALL_ROWS) {  // the deep ring's first slots
      gather_rows(g, v, t, c, true);
      const Loader ld = make_loader(v, t, c);
      const FewRing ring;
      const Rings<4> r;
#pragma unroll
      for (int s = 0; s < FEW_HEAD_SLOTS; ++s) issue_few(ld, ring, r, s, s, n);
      return;
    }
  }
  gather_rows(g, v, t, c);
  const Loader ld = make_loader(v, t, c);
  const Rings<DEPTH> r;
  issue_step(ld, r, -DEPTH, n, 0, 1, 0);
  issue_step(ld, r, 1 - DEPTH, n, 0, 1, 1);
}

template <int DEPTH>
__device__ __forceinline__ void mainloop(const MokGemmResidue& g, const MokGemmTask& t, AccFrag& acc,
                                         const GemmCarry& carry, const MokGemmTask* upcoming, const MokCounters& counters) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31;
  const int half = lane >> 5;
  const Views v = views_of(g, t);
  const int n = v.act.k / K_SLOT;  // the host rejects a contraction length that is not a multiple of 64
  constexpr int XDEPTH = DEPTH + 1;
  const Rings<DEPTH> r;
  const Loader ld = make_loader(v, t, carry);

  // ---- per-fragment LDS read offsets (first block) ------------------------------------
  int xoff[XFRAGS], woff[WFRAGS], xscoff[XFRAGS], wscoff[WFRAGS];
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) {
    const int row = xrow0(wave, b) + r32;
    xoff[b] = row * K_SLOT + 16 * (half ^ swizzle(row));
    xscoff[b] = row * 16;
  }
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) {
    const int wl = wrow0(wave, a) + r32;
    woff[a] = wl * K_SLOT + 16 * (half ^ swizzle(wl));
    wscoff[a] = wl * 4;
  }

  // The accumulator is cleared further down, on each of the two paths by itself (an idle wave's as well: one it left
  // unwritten would be the previous tile's, kept alive across the loop).
  auto clear_accumulator = [&]() {
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a)
#pragma unroll
      for (int b = 0; b < XFRAGS; ++b) acc.v[a][b] = zero_fragment();
  };

  static_assert(DEPTH % 2 == 0, "routed-row pairs start on even steps");
  // steady state, every step issuing: what may be outstanding when step t waits for slot t+1
  constexpr int STEADY_EVEN = DEPTH >= 4 ? (DEPTH - 2) * (W_LOADS + X_LOADS / 2) : 0;            // t even
  constexpr int STEADY_ODD = DEPTH >= 4 ? STEADY_EVEN - X_LOADS / 2 : 0;                         // t odd
  // (the same counts as the run-time formula the tile's last steps use, far from the contraction's end)
  static_assert(DEPTH < 4 || loads_younger_than_slot<DEPTH>(101, 99, 1 << 20) == STEADY_EVEN, "steady wait of an even step");
  static_assert(DEPTH < 4 || loads_younger_than_slot<DEPTH>(102, 100, 1 << 20) == STEADY_ODD, "steady wait of an odd step");

  // ---- rest of the prologue (steps -DEPTH and 1-DEPTH were issued by `prefetch`), then slot 0's operands
#pragma unroll
  for (int u = 2 - DEPTH; u < 0; ++u) issue_step(ld, r, u, n, (u + DEPTH) & ~1, ((u + DEPTH) & ~1) + 1, u + DEPTH);
  // The look-ahead loads go here, behind the prologue's: the waits below count the loads that may still be in flight
  // behind the slot they need, and loads return in order, so one or two more of the youngest only make the next few
  // waits ask for as many more of the oldest.
  if (upcoming->op != 0) stage(g, *upcoming, counters);
  // (with at least DEPTH slots every step up to here has issued its loads: the count is a constant then, and the wait
  // one instruction instead of a computation and a branch table)
  constexpr int ALL_ISSUED = loads_younger_than_slot<DEPTH>(0, -1, 1 << 20);
  if (n >= DEPTH) wait_loads_and_reads<ALL_ISSUED>();
  else wait_loads_and_reads_dyn(loads_younger_than_slot<DEPTH>(0, -1, n));
  wg_barrier();
  auto xnext = [](int b, int by) {  // (b + by) mod XDEPTH for 0 <= b < XDEPTH, 0 <= by <= XDEPTH
    const int c = b + by;
    return c >= XDEPTH ? c - XDEPTH : c;
  };
  if (wave_idle(t, v.w.rows)) {
    // Loader only.  Same loop bounds as the multiplying waves below, one wait + barrier + issue
    // per step, so every wave of the workgroup passes the same number of barriers.
    int xb = 0, wb = 0;
    auto step = [&](int t_) {
      wait_loads_and_reads_dyn(loads_younger_than_slot<DEPTH>(t_ + 1, t_ - 1, n));
      wg_barrier();
      const bool odd_step = t_ & 1;
      issue_step(ld, r, t_, n, odd_step ? xnext(xb, XDEPTH - 2) : xnext(xb, XDEPTH - 1), odd_step ? xnext(xb, XDEPTH - 1) : xb, wb);
      xb = xnext(xb, 1);
      wb = wb + 1 == DEPTH ? 0 : wb + 1;
    };
    int j = 0;
    for (; j + 8 + DEPTH <= n; j += 8)
      for (int s8 = 0; s8 < 8; ++s8) step(j + s8);
    for (; j + 1 < n; j += 2) {
      step(j);
      step(j + 1);
    }
    wg_barrier();
    clear_accumulator();
    return;
  }

  clear_accumulator();
  Operands even, odd;
  int sx[XFRAGS], sw[WFRAGS], sxn[XFRAGS], swn[WFRAGS];
  read_operands(even, r.x(0), r.w(0), xoff, woff);
  read_scales(sx, sw, r.wscale(), r.xscale(), 0, xscoff, wscoff, half);

  // Step j multiplies slot j (already in registers) while it fetches slot j+1's operands from
  // LDS; the barrier in front says slot j+1 has landed for every wave and every wave holds
  // slot j in registers, so slot j's buffers are free.
  //
  // Steady state: groups of eight steps, fully unrolled, as long as every step of the group
  // still has slots to issue.  Weight buffer, scale buffer, scale byte and the slots that carry
  // scale loads are compile-time constants there (the routed-row buffer, modulo DEPTH + 1, is
  // not), so the group is one basic block and the MFMAs stay where they are written, between
  // the LDS reads they overlap with.
  static_assert(8 % DEPTH == 0, "a group of eight slots must start at weight buffer 0");
  int j = 0;
  int xb = 0;  // routed-row buffer of slot j
  for (; j + 8 + DEPTH <= n; j += 8) {
    auto step = [&](auto S_) {
      constexpr int S = decltype(S_)::value;
      constexpr bool ODD = S & 1;
      Operands& cur = ODD ? odd : even;
      Operands& next = ODD ? even : odd;
      __builtin_amdgcn_sched_barrier(0);  // nothing of the previous step sinks below, nothing of this one rises above
      // (the wait and the barrier that free slot j+S's buffers sit behind the step's second MFMA, see below:)
      // slot j+S's buffers are free; so is the routed-row buffer before it (freed a step ago): they take
      // the pair of routed-row slots that starts DEPTH slots ahead of this (even) or the previous (odd) step
      const int xb0 = ODD ? xnext(xb, XDEPTH - 2) : xnext(xb, XDEPTH - 1);
      const int xb1 = ODD ? xnext(xb, XDEPTH - 1) : xb;
      xb = xnext(xb, 1);
      const unsigned char* xnew = r.x(xb);
      const unsigned char* wnew = r.w((S + 1) % DEPTH);
      // The step, MFMA by MFMA.  The first two MFMAs only need registers; the wait and the
      // barrier come behind them, so the matrix pipe has 128 cycles of work while the waves
      // meet.  After the barrier: one LDS unit and one texture-address unit serve the four
      // waves, an LDS read costs the unit about 8 cycles and a 1 KB load about 16, so a wave
      // puts at most two reads and one load between two 64-cycle MFMAs, or the MFMA behind
      // them issues late.  The reads sit in places 2..12 of 16 (the next barrier wants them
      // back), the loads are spread over 2..15.  The scheduler may not move anything from one
      // place to another.
      auto place = [&](auto I_) {
        constexpr int I = decltype(I_)::value;
        constexpr int A = I / XFRAGS, B = I % XFRAGS;
        acc.v[A][B] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(cur.w[A], cur.x[B], acc.v[A][B], 0, 0, ODD ? 2 : 0,
                                                                      sw[A], ODD ? 2 : 0, sx[B]);
        __builtin_amdgcn_sched_barrier(0);  // the MFMA goes first: the pipe is what must not wait
        if constexpr (I == 1) {
          wait_loads_and_reads<ODD ? STEADY_ODD : STEADY_EVEN>();
          wg_barrier();
          __builtin_amdgcn_sched_barrier(0);
        }
        // operand fragment K of the next slot: routed rows first, they are needed by the first MFMAs
        constexpr int K = I == 2 ? 0 : I == 3 ? 1 : I == 5 ? 2 : I == 6 ? 3 : I == 8 ? 4 : I == 9 ? 5 : I == 11 ? 6 : I == 12 ? 7 : -1;
        if constexpr (K >= 0 && K < XFRAGS) next.x[K] = read_frag(xnew, xoff[K]);
        if constexpr (K >= XFRAGS) next.w[K - XFRAGS] = read_frag(wnew, woff[K - XFRAGS]);
        // next pair's scale dwords: read here, shifted into place two MFMAs later, when they have arrived
        if constexpr (ODD && I == 13) read_scales<(S + 1) & 7, false>(sxn, swn, r.wscale(), r.xscale(), j + S + 1, xscoff, wscoff, half);
        if constexpr (ODD && I == 15) shift_scales(sxn, swn, half);
        // this step's loads: 10 on even steps, 8 on odd ones
        if constexpr (DEPTH >= 4) {
          constexpr int LE = I == 2 ? 0 : I == 3 ? 1 : I == 5 ? 2 : I == 6 ? 3 : I == 8 ? 4 : I == 9 ? 5 : I == 11 ? 6 : I == 12 ? 7 : I == 14 ? 8 : I == 15 ? 9 : -1;
          constexpr int LO = (I >= 2 && I % 2 == 0) ? (I - 2) / 2 : I == 15 ? 7 : -1;
          if constexpr (!ODD && LE >= 0) issue_one<false, (S + DEPTH) & 7, LE>(ld, r, j + S + DEPTH, S % DEPTH, xb0, xb1);
          if constexpr (ODD && LO >= 0) issue_one<true, (S + DEPTH) & 7, LO>(ld, r, j + S + DEPTH, S % DEPTH, xb0, xb1);
        } else if constexpr (I == 8) {
          issue_step(ld, r, j + S, n, xb0, xb1, S % DEPTH);
        }
        __builtin_amdgcn_sched_barrier(0);
      };
      place(std::integral_constant<int, 0>{});
      place(std::integral_constant<int, 1>{});
      place(std::integral_constant<int, 2>{});
      place(std::integral_constant<int, 3>{});
      place(std::integral_constant<int, 4>{});
      place(std::integral_constant<int, 5>{});
      place(std::integral_constant<int, 6>{});
      place(std::integral_constant<int, 7>{});
      place(std::integral_constant<int, 8>{});
      place(std::integral_constant<int, 9>{});
      place(std::integral_constant<int, 10>{});
      place(std::integral_constant<int, 11>{});
      place(std::integral_constant<int, 12>{});
      place(std::integral_constant<int, 13>{});
      place(std::integral_constant<int, 14>{});
      place(std::integral_constant<int, 15>{});
      __builtin_amdgcn_sched_barrier(0);
      if (ODD) {
#pragma unroll
        for (int b = 0; b < XFRAGS; ++b) sx[b] = sxn[b];
#pragma unroll
        for (int a = 0; a < WFRAGS; ++a) sw[a] = swn[a];
      }
    };
    step(std::integral_constant<int, 0>{});
    step(std::integral_constant<int, 1>{});
    step(std::integral_constant<int, 2>{});
    step(std::integral_constant<int, 3>{});
    step(std::integral_constant<int, 4>{});
    step(std::integral_constant<int, 5>{});
    step(std::integral_constant<int, 6>{});
    step(std::integral_constant<int, 7>{});
  }

  // Remaining slots (fewer than 8 + DEPTH), same steps with run-time slot numbers.  The MFMA
  // chain is straight-line code: past the last slot `advance` still runs (it reads buffers
  // nobody uses), which keeps control flow out of the accumulator's live range.
  int wb = 0;  // weight buffer of slot j (j is a multiple of 8 here)
  auto advance = [&](int t_, Operands& next) {
    wait_loads_and_reads_dyn(loads_younger_than_slot<DEPTH>(t_ + 1, t_ - 1, n));
    wg_barrier();
    const bool odd_step = t_ & 1;
    issue_step(ld, r, t_, n, odd_step ? xnext(xb, XDEPTH - 2) : xnext(xb, XDEPTH - 1), odd_step ? xnext(xb, XDEPTH - 1) : xb, wb);
    xb = xnext(xb, 1);
    wb = wb + 1 == DEPTH ? 0 : wb + 1;
    read_operands(next, r.x(xb), r.w(wb), xoff, woff);
  };
  for (; j + 1 < n; j += 2) {
    advance(j, odd);
    mma_step<false>(even, sx, sw, acc);
    advance(j + 1, even);
    read_scales(sxn, swn, r.wscale(), r.xscale(), j + 2, xscoff, wscoff, half);
    mma_step<true>(odd, sx, sw, acc);
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b) sx[b] = sxn[b];
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) sw[a] = swn[a];
  }
  if (n & 1) mma_step<false>(even, sx, sw, acc);  // a last single slot is already in registers
  wg_barrier();  // every wave holds its last operands in registers: the ring is free
}


// ---- tiles with little to multiply (mok::tile_placement) ----------------------------------------------------------
// An expert's rows past its last full tile (1 to 64 of them) and the columns past the last full column tile (64 of
// them when the width is 2880) would keep two of the four waves busy with a 128 x 128 share that is mostly padding,
// for as long as a full tile takes.  Such a tile is multiplied in the other placement: every wave takes 64 routed
// rows and one or two pairs of weight fragments, a quarter or half of the full tile's MFMAs spread over all four
// SIMDs, and the tile takes as long as its loads do.  Rings, loader, waits and barriers are the full tile's (the
// loader does not know the difference); the loop is the plain two-stage one the full tile ends with.
struct SmallOperands {
  v8i x[2], w[4];
};

template <int DEPTH, int FRAGS>  // FRAGS: the weight fragments that are multiplied, bit a
__device__ __forceinline__ void mainloop_small(const MokGemmResidue& g, const MokGemmTask& t, int placement, AccFrag& acc,
                                               const GemmCarry& carry, const MokGemmTask* upcoming, const MokCounters& counters) {
  const int tid = fresh_tid();  // nothing of this path is to be computed ahead and kept across full tiles
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31;
  const int half = lane >> 5;
  const Views v = views_of(g, t);
  const int n = v.act.k / K_SLOT;
  constexpr int XDEPTH = DEPTH + 1;
  const Rings<DEPTH> r;
  const Loader ld = make_loader(v, t, carry);
  const SmallPlacement sp = small_placement(placement, wave);
  auto used = [](int a) { return (FRAGS >> a & 1) != 0; };

  int xoff[2], xscoff[2], woff[4], wscoff[4];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int row = sp.xr0 + 32 * b + r32;
    xoff[b] = row * K_SLOT + 16 * (half ^ swizzle(row));
    xscoff[b] = row * 16;
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {
    const int wl = sp.wr[a] + r32;
    woff[a] = wl * K_SLOT + 16 * (half ^ swizzle(wl));
    wscoff[a] = wl * 4;
  }
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
      if (used(a)) acc.v[a][b] = zero_fragment();

  // the prologue of the full tile: steps -DEPTH and 1 - DEPTH were issued by `prefetch`
#pragma unroll
  for (int u = 2 - DEPTH; u < 0; ++u) issue_step(ld, r, u, n, (u + DEPTH) & ~1, ((u + DEPTH) & ~1) + 1, u + DEPTH);
  if (upcoming->op != 0) stage(g, *upcoming, counters);
  // (with at least DEPTH slots every step up to here has issued its loads: the count is a constant then, and the wait
  // one instruction instead of a computation and a branch table)
  constexpr int ALL_ISSUED = loads_younger_than_slot<DEPTH>(0, -1, 1 << 20);
  if (n >= DEPTH) wait_loads_and_reads<ALL_ISSUED>();
  else wait_loads_and_reads_dyn(loads_younger_than_slot<DEPTH>(0, -1, n));
  wg_barrier();

  auto xnext = [](int b, int by) {
    const int c = b + by;
    return c >= XDEPTH ? c - XDEPTH : c;
  };
  auto read_operands_small = [&](SmallOperands& o, const unsigned char* xbuf, const unsigned char* wbuf) {
#pragma unroll
    for (int b = 0; b < 2; ++b) o.x[b] = read_frag(xbuf, xoff[b]);
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (used(a)) o.w[a] = read_frag(wbuf, woff[a]);
  };
  // block scales of the pair of slots that starts at slot j (j even), as read_scales does for the full tile
  auto read_scales_small = [&](int (&sx_)[2], int (&sw_)[4], int j) {
    const int c = (j & 7) >> 1;
    const unsigned char* xbuf = r.xscale() + ((j >> 3) & 1) * (TILE_X * 16);
    const unsigned char* wbuf = r.wscale() + c * (TILE_W * 4);
#pragma unroll
    for (int b = 0; b < 2; ++b) sx_[b] = (int)(*reinterpret_cast<const uint32_t*>(xbuf + 4 * c + xscoff[b]) >> (8 * half));
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (used(a)) sw_[a] = (int)(*reinterpret_cast<const uint32_t*>(wbuf + wscoff[a]) >> (8 * half));
  };
  SmallOperands even, odd;
  int sx[2], sw[4], sxn[2], swn[4];
  auto multiply = [&](auto ODD_, const SmallOperands& o) {
    constexpr bool ODD = decltype(ODD_)::value;
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (used(a)) {
#pragma unroll
        for (int b = 0; b < 2; ++b)
          acc.v[a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(o.w[a], o.x[b], acc.v[a][b], 0, 0, ODD ? 2 : 0, sw[a],
                                                                        ODD ? 2 : 0, sx[b]);
      }
  };
  read_operands_small(even, r.x(0), r.w(0));
  read_scales_small(sx, sw, 0);
  int xb = 0, wb = 0;
  auto advance = [&](int t_, SmallOperands& next) {
    wait_loads_and_reads_dyn(loads_younger_than_slot<DEPTH>(t_ + 1, t_ - 1, n));
    wg_barrier();
    const bool odd_step = t_ & 1;
    issue_step(ld, r, t_, n, odd_step ? xnext(xb, XDEPTH - 2) : xnext(xb, XDEPTH - 1), odd_step ? xnext(xb, XDEPTH - 1) : xb, wb);
    xb = xnext(xb, 1);
    wb = wb + 1 == DEPTH ? 0 : wb + 1;
    read_operands_small(next, r.x(xb), r.w(wb));
  };
  int j = 0;
  for (; j + 1 < n; j += 2) {
    advance(j, odd);
    multiply(std::false_type{}, even);
    advance(j + 1, even);
    read_scales_small(sxn, swn, j + 2);
    multiply(std::true_type{}, odd);
#pragma unroll
    for (int b = 0; b < 2; ++b) sx[b] = sxn[b];
#pragma unroll
    for (int a = 0; a < 4; ++a)
      if (used(a)) sw[a] = swn[a];
  }
  if (n & 1) multiply(std::false_type{}, even);
  wg_barrier();  // every wave holds its last operands in registers: the ring is free
}



// The mainloop of a tile of at most 64 rows in the deep ring (ring depth 4 and up; mainloop_small<DEPTH, SMALL_ROWS_FRAGS>
// otherwise): the small placement's fragments a = 0 and a = 2, two routed-row fragments, four MFMAs a step.
__device__ __forceinline__ void mainloop_few_rows(const MokGemmResidue& g, const MokGemmTask& t, AccFrag& acc, const GemmCarry& carry,
                                                  const MokGemmTask* upcoming, const MokCounters& counters) {
  const int tid = fresh_tid();  // nothing of this path is to be computed ahead and kept across full tiles
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r32 = lane & 31;
  const int half = lane >> 5;
  const Views v = views_of(g, t);
  const int n = v.act.k / K_SLOT;
  const FewRing ring;
  const Rings<4> r;
  const Loader ld = make_loader(v, t, carry);
  const SmallPlacement sp = small_placement(TILE_SMALL_ROWS, wave);
  int xoff[2], xscoff[2], woff[2], wscoff[2];
#pragma unroll
  for (int b = 0; b < 2; ++b) {
    const int row = 32 * b + r32;
    xoff[b] = BUF_BYTES + row * K_SLOT + 16 * (half ^ swizzle(row));
    xscoff[b] = row * 16;
  }
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    const int wl = sp.wr[2 * a] + r32;
    woff[a] = wl * K_SLOT + 16 * (half ^ swizzle(wl));
    wscoff[a] = wl * 4;
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b) acc.v[2 * a][b] = zero_fragment();

  // slots 0 .. FEW_HEAD_SLOTS - 1 were asked for by `prefetch`; the rest of the ring now
#pragma unroll
  for (int s = FEW_HEAD_SLOTS; s < FEW_DEPTH; ++s) issue_few(ld, ring, r, s, s, n);
  if (upcoming->op != 0) stage(g, *upcoming, counters);
  wait_few(few_younger(0, -1, n));
  wg_barrier();

  struct FewOperands {
    v8i x[2], w[2];
  } even, odd;
  int sx[2], sw[2], sxn[2], swn[2];
  auto read_operands_few = [&](FewOperands& o, const unsigned char* slot) {
#pragma unroll
    for (int b = 0; b < 2; ++b) o.x[b] = read_frag(slot, xoff[b]);
#pragma unroll
    for (int a = 0; a < 2; ++a) o.w[a] = read_frag(slot, woff[a]);
  };
  auto read_scales_few = [&](int (&sx_)[2], int (&sw_)[2], int j) {  // of the pair of slots that starts at slot j (j even)
    const int c = (j & 7) >> 1;
    const unsigned char* xbuf = r.xscale() + ((j >> 3) & 1) * (TILE_X * 16);
    const unsigned char* wbuf = r.wscale() + c * (TILE_W * 4);
#pragma unroll
    for (int b = 0; b < 2; ++b) sx_[b] = (int)(*reinterpret_cast<const uint32_t*>(xbuf + 4 * c + xscoff[b]) >> (8 * half));
#pragma unroll
    for (int a = 0; a < 2; ++a) sw_[a] = (int)(*reinterpret_cast<const uint32_t*>(wbuf + wscoff[a]) >> (8 * half));
  };
  auto multiply = [&](auto ODD_, const FewOperands& o) {
    constexpr bool ODD = decltype(ODD_)::value;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
        acc.v[2 * a][b] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(o.w[a], o.x[b], acc.v[2 * a][b], 0, 0, ODD ? 2 : 0, sw[a],
                                                                          ODD ? 2 : 0, sx[b]);
  };
  read_operands_few(even, ring.slot(0));
  read_scales_few(sx, sw, 0);
  int pos = 0;  // ring position of slot t_ in `advance`
  // step t_: slot t_ + 1 has landed for every wave and every wave holds slot t_ in registers, whose place takes slot
  // t_ + FEW_DEPTH
  auto advance = [&](int t_, FewOperands& next) {
    wait_few(few_younger(t_ + 1, t_ - 1, n));
    wg_barrier();
    issue_few(ld, ring, r, t_ + FEW_DEPTH, pos, n);
    pos = pos + 1 == FEW_DEPTH ? 0 : pos + 1;
    read_operands_few(next, ring.slot(pos));
  };
  int j = 0;
  for (; j + 1 < n; j += 2) {
    advance(j, odd);
    multiply(std::false_type{}, even);
    advance(j + 1, even);
    read_scales_few(sxn, swn, j + 2);
    multiply(std::true_type{}, odd);
#pragma unroll
    for (int b = 0; b < 2; ++b) sx[b] = sxn[b];
#pragma unroll
    for (int a = 0; a < 2; ++a) sw[a] = swn[a];
  }
  if (n & 1) multiply(std::false_type{}, even);
  wg_barrier();  // every wave holds its last operands in registers: the ring is free
}

// bf16 epilogue of the down op.  The accumulator is transposed through the arena buffers (idle
// by now; the head may already hold the next tile's first slots) so that the global stores
// are 16 bytes per lane and 512 contiguous bytes per routed row; an arena too small for the
// whole tile stages the two 128-row halves one after the other.  An arena that cannot hold
// half a tile (depth 2) falls back to 8-byte stores straight from the registers.
constexpr int Y_PITCH = TILE_W * 2 + 16;  // bytes per staged row: 256 bf16 + pad against bank conflicts

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32, nearest even
}

template <int DEPTH, int FRAGS>  // FRAGS: 0 for a full tile, else the fragments a small tile's waves hold
__device__ __forceinline__ void store_down(const MokGemmResidue& g, const MokGemmTask& t, int placement, const AccFrag& acc) {
  constexpr int ARENA_BYTES = (2 * DEPTH - 3) * BUF_BYTES;
  const int tid = fresh_tid();
  const int lane = tid & 63;
  const int wave = tid >> 6;
  constexpr bool small = FRAGS != 0;
  const SmallPlacement sp = small_placement(placement, __builtin_amdgcn_readfirstlane(wave));
  const bool idle = !small && wave_idle(t, g.w_down.rows);  // this wave's accumulator holds nothing
  if constexpr (ARENA_BYTES < TILE_X / 2 * Y_PITCH) {
    if (small) {
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        const int row = t.row_begin + sp.xr0 + 32 * b + (lane & 31);
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          if (!(FRAGS >> a & 1)) continue;
          const v16f f = from_acc(acc.v[a][b]);
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            const int col = t.col_begin + sp.wr[a] + 8 * q + 4 * (lane >> 5);
            if (row < t.row_end && col < g.w_down.rows) {
              uint2 pk;
              pk.x = pack_bf16x2(f[4 * q + 0], f[4 * q + 1]);
              pk.y = pack_bf16x2(f[4 * q + 2], f[4 * q + 3]);
              *reinterpret_cast<uint2*>(g.y + (int64_t)row * g.ld_y + col) = pk;
            }
          }
        }
      }
      return;
    }
    if (idle) return;
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b) {
      const int row = t.row_begin + xrow0(wave, b) + (lane & 31);
#pragma unroll
      for (int a = 0; a < WFRAGS; ++a) {
        const v16f f = from_acc(acc.v[a][b]);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int col = t.col_begin + wrow0(wave, a) + 8 * q + 4 * (lane >> 5);
          if (row < t.row_end && col < g.w_down.rows) {
            uint2 pk;
            pk.x = pack_bf16x2(f[4 * q + 0], f[4 * q + 1]);
            pk.y = pack_bf16x2(f[4 * q + 2], f[4 * q + 3]);
            *reinterpret_cast<uint2*>(g.y + (int64_t)row * g.ld_y + col) = pk;
          }
        }
      }
    }
  } else {
    constexpr int PASSES = TILE_X * Y_PITCH <= ARENA_BYTES ? 1 : 2;
    constexpr int ROWS = TILE_X / PASSES;  // rows staged per pass
    unsigned char* stage = pipelink_smem + pipelink_mok_gemm_arena();
    const int chunk = lane & 31;                                  // 8 columns = 16 bytes
    const bool col_ok = t.col_begin + chunk * 8 < g.w_down.rows;  // column extents are multiples of 32
#pragma unroll
    for (int pass = 0; pass < PASSES; ++pass) {
      if (small) {
        // every wave's 64 rows lie in one pass; a tile of at most 64 rows has nothing in a second pass
        if (PASSES == 2 && pass == 1 && placement == TILE_SMALL_ROWS) break;
        if (PASSES == 1 || (sp.xr0 >= ROWS) == (pass == 1)) {
#pragma unroll
          for (int b = 0; b < 2; ++b) {
            unsigned char* rowp = stage + (sp.xr0 + 32 * b - pass * ROWS + (lane & 31)) * Y_PITCH;
#pragma unroll
            for (int a = 0; a < 4; ++a) {
              if (!(FRAGS >> a & 1)) continue;
              const v16f f = from_acc(acc.v[a][b]);
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                const int col = sp.wr[a] + 8 * q + 4 * (lane >> 5);
                uint2 pk;
                pk.x = pack_bf16x2(f[4 * q + 0], f[4 * q + 1]);
                pk.y = pack_bf16x2(f[4 * q + 2], f[4 * q + 3]);
                *reinterpret_cast<uint2*>(rowp + col * 2) = pk;
              }
            }
          }
        }
      } else if (!idle && (PASSES == 1 || wave_x(wave) == pass)) {
#pragma unroll
        for (int b = 0; b < XFRAGS; ++b) {
          unsigned char* rowp = stage + (xrow0(wave, b) - pass * ROWS + (lane & 31)) * Y_PITCH;
#pragma unroll
          for (int a = 0; a < WFRAGS; ++a) {
            const v16f f = from_acc(acc.v[a][b]);
#pragma unroll
            for (int q = 0; q < 4; ++q) {
              const int col = wrow0(wave, a) + 8 * q + 4 * (lane >> 5);
              uint2 pk;
              pk.x = pack_bf16x2(f[4 * q + 0], f[4 * q + 1]);
              pk.y = pack_bf16x2(f[4 * q + 2], f[4 * q + 3]);
              *reinterpret_cast<uint2*>(rowp + col * 2) = pk;
            }
          }
        }
      }
      __syncthreads();
#pragma unroll 4
      for (int it = 0; it < ROWS / WAVES / 2; ++it) {
        const int srow = wave * (ROWS / WAVES) + it * 2 + (lane >> 5);
        const int row = t.row_begin + pass * ROWS + srow;
        if (row < t.row_end && col_ok) {
          const uint4 v = *reinterpret_cast<const uint4*>(stage + srow * Y_PITCH + chunk * 16);
          *reinterpret_cast<uint4*>(g.y + (int64_t)row * g.ld_y + t.col_begin + chunk * 8) = v;
        }
      }
      __syncthreads();  // the arena is reused by the next pass or the next tile's loads
    }
  }
}

}  // namespace mok_gemm_owner

extern "C" __device__ void mok_gemm_init(const void* view) { (void)view; }
// Nothing to give back: the owner holds no barriers or tensor memory of its own (campaigns/mok/port/gemm/gemm_abi.h:52-54
// exports init, fini and fwd; init and fini are where the reference sets up and frees its mbarriers and TMEM columns).
extern "C" __device__ void mok_gemm_fini(const void* view) { (void)view; }

static __device__ __forceinline__ const MokGemmResidue& mok_gemm_residue(const void* view) {
  return *static_cast<const MokGemmResidue*>(static_cast<const pipelink_host_view*>(view)->residue);
}

// The placement of the task's tile (mok::TILE_FULL, or one of the small ones): which exports the caller uses for it.
extern "C" __device__ int mok_gemm_placement(const void* view, const MokGemmTask* task) {
  return mok_gemm_owner::placement_of(mok_gemm_residue(view), *task);
}

// Looks ahead to a task outside a mainloop (a workgroup's first tile): asks for the task's row tokens and readiness
// counter.  The caller waits for its loads and passes a workgroup barrier before it calls mok_gemm_ready / _prefetch.
extern "C" __device__ void mok_gemm_stage(const void* view, const MokGemmTask* task, const MokCounters* counters) {
  mok_gemm_owner::stage(mok_gemm_residue(view), *task, *counters);
}

// True if the rows the staged task reads were complete when it was staged (always, for a task that depends on none).
extern "C" __device__ bool mok_gemm_ready(const void* view, const MokGemmTask* task, const MokCounters* counters) {
  (void)view;
  return mok_gemm_owner::staged_ready(*task, *counters);
}

// Waits (bounded) until the rows the task reads are complete; raises MOK_STATUS_WAIT_GAVE_UP in *counters->status
// if they are not after 2^14 polls (or at once, if a wait of the launch has given up before).  Must not be called while the workgroup holds a tile whose results others wait for.
extern "C" __device__ void mok_gemm_wait(const void* view, const MokGemmTask* task, const MokCounters* counters) {
  (void)view;
  mok_gemm_owner::wait_rows(*task, *counters);
}

// Starts the loads of a tile's first two slots and leaves the gathered row offsets in *carry.  The task must have been
// staged, and the rows it reads must be complete (mok_gemm_ready / mok_gemm_wait).
// Only touches the head buffers: the caller may run it between the previous tile's mainloop
// and that tile's epilogue.
extern "C" __device__ void mok_gemm_prefetch(const void* view, const MokGemmTask* task, mok::GemmCarry* carry) {
  const auto& g = mok_gemm_residue(view);
  switch (pipelink_mok_gemm_depth()) {  // a link-time constant: one case survives
    case 2: mok_gemm_owner::prefetch<2>(g, *task, *carry); break;
    default: mok_gemm_owner::prefetch<4>(g, *task, *carry); break;
  }
}

// Runs the mainloop of one tile whose prefetch has been issued (same task, same carry) and
// leaves the fp32 accumulator in *acc: for the activation owner (gate/up op) or for
// mok_gemm_store (down op).  `upcoming`, unless its op is 0, is the task this workgroup runs next: it is staged
// (see mok_gemm_stage) behind the tile's first loads, and is ready for mok_gemm_ready / _prefetch when the call returns.
// *phase counts the tiles this workgroup has multiplied.
extern "C" __device__ void mok_gemm_fwd(const void* view, const MokGemmTask* task, const MokCounters* counters,
                                        uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry,
                                        const MokGemmTask* upcoming) {
  const auto& g = mok_gemm_residue(view);
  switch (pipelink_mok_gemm_depth()) {
    case 2: mok_gemm_owner::mainloop<2>(g, *task, *acc, *carry, upcoming, *counters); break;
    default: mok_gemm_owner::mainloop<4>(g, *task, *acc, *carry, upcoming, *counters); break;
  }
  ++*phase;
}

// mok_gemm_fwd for a tile in the small placement (mok::tile_placement of the task's extent is not TILE_FULL): the
// caller tells the two apart, and hands the accumulator to mok_act_fwd_small / mok_gemm_store_small.
extern "C" __device__ void mok_gemm_fwd_small(const void* view, const MokGemmTask* task, const MokCounters* counters,
                                              uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry,
                                              const MokGemmTask* upcoming) {
  const auto& g = mok_gemm_residue(view);
  const int placement = mok_gemm_owner::placement_of(g, *task);
  const bool gate_up = task->op == MOK_GEMM_FWD_ROUTED_GATE_UP;
  const int frags = placement == mok::TILE_SMALL_ROWS ? mok::SMALL_ROWS_FRAGS
                    : gate_up ? mok::SMALL_COLS_FRAGS_GATE_UP : mok::SMALL_COLS_FRAGS_DOWN;
#define PL_SMALL(D, F) case F: mok_gemm_owner::mainloop_small<D, F>(g, *task, placement, *acc, *carry, upcoming, *counters); break;
  switch (pipelink_mok_gemm_depth()) {
    case 2:
      switch (frags) { PL_SMALL(2, mok::SMALL_ROWS_FRAGS) PL_SMALL(2, mok::SMALL_COLS_FRAGS_GATE_UP) PL_SMALL(2, mok::SMALL_COLS_FRAGS_DOWN) }
      break;
    default:
      if (placement == mok::TILE_SMALL_ROWS) {  // (the deep ring needs the arena of depth 4; mok_gemm_prefetch decides alike)
        mok_gemm_owner::mainloop_few_rows(g, *task, *acc, *carry, upcoming, *counters);
        break;
      }
      switch (frags) { PL_SMALL(4, mok::SMALL_COLS_FRAGS_GATE_UP) PL_SMALL(4, mok::SMALL_COLS_FRAGS_DOWN) }
      break;
  }
#undef PL_SMALL
  ++*phase;
}

// Down op only: rounds the accumulator to bf16 and stores the tile of y.
extern "C" __device__ void mok_gemm_store(const void* view, const MokGemmTask* task, const mok::AccFrag* acc) {
  const auto& g = mok_gemm_residue(view);
  switch (pipelink_mok_gemm_depth()) {
    case 2: mok_gemm_owner::store_down<2, 0>(g, *task, mok::TILE_FULL, *acc); break;
    default: mok_gemm_owner::store_down<4, 0>(g, *task, mok::TILE_FULL, *acc); break;
  }
}

// mok_gemm_store for a tile in the small placement.
extern "C" __device__ void mok_gemm_store_small(const void* view, const MokGemmTask* task, const mok::AccFrag* acc) {
  const auto& g = mok_gemm_residue(view);
  const int placement = mok_gemm_owner::placement_of(g, *task);
#define PL_STORE(D)                                                                                                  \
  if (placement == mok::TILE_SMALL_ROWS) mok_gemm_owner::store_down<D, mok::SMALL_ROWS_FRAGS>(g, *task, placement, *acc); \
  else mok_gemm_owner::store_down<D, mok::SMALL_COLS_FRAGS_DOWN>(g, *task, placement, *acc);
  switch (pipelink_mok_gemm_depth()) {
    case 2: PL_STORE(2) break;
    default: PL_STORE(4) break;
  }
#undef PL_STORE
}
#else  // PIPELINK_EMIT: host-evaluated annotations only
#include "../include/mok_abi.h"
#endif

PL_STAGE("mok.gemm", "0.1.0");
PL_PARAMS(MokGemmResidue);
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {{"pipelink_mok_precision", 1}});  // MXFP8 (campaigns/mok/port/include/mok_abi.h: MOK_PRECISION_MXFP8)
PL_EXPORT(mok_gemm_init, mok_gemm_init, "extern \"C\" __device__ void mok_gemm_init(const void* view);");
PL_EXPORT(mok_gemm_fini, mok_gemm_fini, "extern \"C\" __device__ void mok_gemm_fini(const void* view);");
PL_EXPORT(mok_gemm_stage, mok_gemm_stage,
          "extern \"C\" __device__ void mok_gemm_stage(const void* view, const MokGemmTask* task, const MokCounters* counters);");
PL_EXPORT(mok_gemm_ready, mok_gemm_ready,
          "extern \"C\" __device__ bool mok_gemm_ready(const void* view, const MokGemmTask* task, const MokCounters* counters);");
PL_EXPORT(mok_gemm_wait, mok_gemm_wait,
          "extern \"C\" __device__ void mok_gemm_wait(const void* view, const MokGemmTask* task, const MokCounters* counters);");
PL_EXPORT(mok_gemm_prefetch, mok_gemm_prefetch,
          "extern \"C\" __device__ void mok_gemm_prefetch(const void* view, const MokGemmTask* task, mok::GemmCarry* carry);");
PL_EXPORT(mok_gemm_fwd, mok_gemm_fwd,
          "extern \"C\" __device__ void mok_gemm_fwd(const void* view, const MokGemmTask* task, "
          "const MokCounters* counters, uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry, "
          "const MokGemmTask* upcoming);");
PL_EXPORT(mok_gemm_store, mok_gemm_store,
          "extern \"C\" __device__ void mok_gemm_store(const void* view, const MokGemmTask* task, const mok::AccFrag* acc);");
PL_EXPORT(mok_gemm_placement, mok_gemm_placement,
          "extern \"C\" __device__ int mok_gemm_placement(const void* view, const MokGemmTask* task);");
PL_EXPORT(mok_gemm_fwd_small, mok_gemm_fwd_small,
          "extern \"C\" __device__ void mok_gemm_fwd_small(const void* view, const MokGemmTask* task, "
          "const MokCounters* counters, uint32_t* phase, mok::AccFrag* acc, const mok::GemmCarry* carry, "
          "const MokGemmTask* upcoming);");
PL_EXPORT(mok_gemm_store_small, mok_gemm_store_small,
          "extern \"C\" __device__ void mok_gemm_store_small(const void* view, const MokGemmTask* task, const mok::AccFrag* acc);");
PL_SERVE(gemm_init, "mok_gemm_init");
PL_SERVE(gemm_fini, "mok_gemm_fini");
PL_SERVE(gemm_stage, "mok_gemm_stage");
PL_SERVE(gemm_ready, "mok_gemm_ready");
PL_SERVE(gemm_wait, "mok_gemm_wait");
PL_SERVE(gemm_prefetch, "mok_gemm_prefetch");
PL_SERVE(gemm_fwd, "mok_gemm_fwd");
PL_SERVE(gemm_store, "mok_gemm_store");
PL_SERVE(gemm_placement, "mok_gemm_placement");
PL_SERVE(gemm_fwd_small, "mok_gemm_fwd_small");
PL_SERVE(gemm_store_small, "mok_gemm_store_small");
// head, live for the whole kernel: the first two 16 KB buffers of the routed-row ring and of the weight
// ring, four 1 KB buffers of weight scales, two 4 KB buffers of routed-row scales, the staged task's row tokens (1 KB)
// and readiness counter (256 B)
PL_CLAIM("pipelink_mok_gemm_head", "smem", 4 * 16384 + 4096 + 8192 + 1024 + 256, 1024, "kernel");
// arena, live during the GEMM phase: the other buffers of the two rings -- depth + 1 - 2 routed-row
// buffers and depth - 2 weight buffers, (2 * depth - 3) x 16 KB
PL_CLAIM_RING("pipelink_mok_gemm_arena", "smem", -3 * 16384, "pipelink_mok_gemm_depth", 32768, 1024, "phase:instr_gemm");
PL_USES("pipelink_mok_gemm_head");
PL_USES("pipelink_mok_gemm_depth");
PL_USES("pipelink_mok_gemm_arena");
// host contract (the reference's PL_HOST_* block, campaigns/mok/port/gemm/gemm.cu:383-479): provider entry points
// pipelink_params_*_mok_gemm, the records it reports, the caller's tensors
PL_HOST_GROUP("mok.gemm.params", "mok_gemm");
PL_HOST_ABI_TYPE(1, MokGemmResidue);
PL_HOST_ABI_TYPE(4, MokMxView);
MOK_HOST_SCALARS();
PL_HOST_CHANNEL(1, "x_q", 8, "read", "mok.num_local_tokens, mok.ld_q_h", false);
PL_HOST_CHANNEL(2, "x_sc", 8, "read", "mok.num_local_tokens, mok.ld_sc_h", false);
PL_HOST_CHANNEL(3, "w_gate_q", 8, "read", "mok.num_local_experts, floor(mok.hidden,64), mok.intermediate, 64", false);
PL_HOST_CHANNEL(4, "w_gate_sc", 8, "read", "mok.num_local_experts, ceil(mok.hidden,128), mok.intermediate, 4", false);
PL_HOST_CHANNEL(5, "w_up_q", 8, "read", "mok.num_local_experts, floor(mok.hidden,64), mok.intermediate, 64", false);
PL_HOST_CHANNEL(6, "w_up_sc", 8, "read", "mok.num_local_experts, ceil(mok.hidden,128), mok.intermediate, 4", false);
PL_HOST_CHANNEL(7, "w_down_q", 8, "read", "mok.num_local_experts, floor(mok.intermediate,64), mok.hidden, 64", false);
PL_HOST_CHANNEL(8, "w_down_sc", 8, "read", "mok.num_local_experts, ceil(mok.intermediate,128), mok.hidden, 4", false);
PL_HOST_CHANNEL(9, "hidden_q", 8, "read", "mok.routed_rows, mok.ld_q_i", false);
PL_HOST_CHANNEL(10, "hidden_sc", 8, "read", "mok.routed_rows, mok.ld_sc_i", false);
PL_HOST_CHANNEL(11, "y", 16, "write", "mok.routed_rows, mok.hidden", false);
PL_HOST_CHANNEL(12, "row_token", 32, "read", "mok.routed_rows", true);  // left out: routed rows are tokens
PL_FACT("mok.gemm.TILE_X", 256);
PL_FACT("mok.gemm.TILE_W", 256);
PL_FACT("mok.gemm.K_SLOT", 64);
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
