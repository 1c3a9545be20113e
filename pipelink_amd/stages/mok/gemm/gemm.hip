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
// Ring: `depth` LDS slots of 66 KB.  A slot holds 128 contraction bytes of 256 routed rows
// and of 256 weight rows, row-major (one 128-byte cache line per row), followed by one
// dword of block scales (4 x e8m0) per row.  One global_load_lds_dwordx4 moves 8 rows:
// eight lanes cover the 128 contiguous bytes of a row, so every L2 request is a full line.
// The eight 16-byte chunks of a row are stored at position chunk ^ ((row / 2) % 8), which
// makes a fragment read (32 consecutive rows, one chunk each) touch 16 different 16-byte
// bank groups per 16 lanes.  The depth is a link-time handle; the ring offset inside the
// workgroup's dynamic LDS is another.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include "../include/mok_device.hpp"

extern "C" __device__ int pipelink_mok_gemm_depth();  // ring slots (2 or 3), bound at link time
extern "C" __device__ int pipelink_mok_gemm_arena();  // byte offset of the ring in dynamic LDS

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mok_gemm_owner {
using namespace mok;

constexpr int WAVES = THREADS / 64;
constexpr int X_GROUPS = TILE_X / 8 / WAVES;  // 8-row load groups per wave (4)
constexpr int W_GROUPS = TILE_W / 8 / WAVES;  // (4)
constexpr int LOADS_PER_SLOT = X_GROUPS + W_GROUPS + 1;  // + one dword of scales per lane

// Addresses are a wave-uniform base (kept in scalar registers) plus a 32-bit lane offset: one
// operand of one expert is far below 4 GiB, and 8 + 1 offsets cost half the vector registers
// of 9 pointers.
struct Loader {
  const uint8_t* xbase;           // activations (all rows)
  const uint8_t* wbase;           // this expert's weight matrix (gate or up or down, by wave)
  const uint8_t* scbase;          // scale matrix this thread's row belongs to
  uint32_t xsrc[X_GROUPS];        // this lane's 16 bytes of its row in each group, at k = 0
  uint32_t wsrc[W_GROUPS];
  uint32_t scsrc;                 // scale row of this thread's row (threads 0..255 rows, 256..511 weights)
  int chunk_byte;                 // byte offset inside the 128-byte line this lane fetches in even groups
  int xdst, wdst, scdst;          // slot-relative LDS byte offsets of the wave's first group
};

__device__ __forceinline__ int swizzle(int row) { return (row >> 1) & 7; }

// Issue one slot.  k_left = contraction bytes from this slot's start to the end of the row:
// the last slot of a K that is not a multiple of 128 only fetches the chunks that exist.
__device__ __forceinline__ void issue_slot(const Loader& ld, unsigned char* slot, int kbyte, int k_left) {
  // group j starts at tile row 8 * (4 * wave + j): odd groups flip bit 2 of the swizzle, so
  // the lane's chunk there is the even-group chunk with bit 2 (64 bytes) flipped
#pragma unroll
  for (int j = 0; j < X_GROUPS; ++j)
    if ((ld.chunk_byte ^ ((j & 1) << 6)) < k_left) load16_to_lds(ld.xbase + kbyte + ld.xsrc[j], slot + ld.xdst + j * 1024);
#pragma unroll
  for (int j = 0; j < W_GROUPS; ++j)
    if ((ld.chunk_byte ^ ((j & 1) << 6)) < k_left) load16_to_lds(ld.wbase + kbyte + ld.wsrc[j], slot + ld.wdst + j * 1024);
  load4_to_lds(ld.scbase + (kbyte >> 5) + ld.scsrc, slot + ld.scdst);
}

// MFMA 32x32x64 f8f6f4 operand of lane (row = lane % 32, half = lane / 32): registers 0-3
// hold 16 bytes of the step's first 32-element block, registers 4-7 16 bytes of its second
// block; the scale of block 0 is taken from lanes 0-31 and that of block 1 from lanes 32-63
// (measured on gfx950 with a one-instruction probe).  So in 64-byte step s of a slot a lane
// reads chunks 4s + half and 4s + half + 2 of its row; with the XOR swizzle these are the
// step-0 offsets with bit 6 (step) and bit 5 (second block) flipped.
__device__ __forceinline__ v8i read_frag(const unsigned char* slot, int off) {
  const v4i lo = *reinterpret_cast<const v4i*>(slot + off);
  const v4i hi = *reinterpret_cast<const v4i*>(slot + (off ^ 32));
  v8i r;
  r.s0 = lo.x; r.s1 = lo.y; r.s2 = lo.z; r.s3 = lo.w;
  r.s4 = hi.x; r.s5 = hi.y; r.s6 = hi.z; r.s7 = hi.w;
  return r;
}

// Workgroup barrier without the release/acquire fence of __syncthreads(): a fence would
// drain every outstanding global->LDS load (vmcnt(0)) and serialise the ring.  Ordering of
// the LDS traffic is by the explicit s_waitcnt in front of it.
__device__ __forceinline__ void wg_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 0xF) | ((N >> 4) << 14));
}

template <bool ODD>
__device__ __forceinline__ void mma_step(const unsigned char* slot, const int (&xoff)[XFRAGS],
                                         const int (&woff)[WFRAGS], const int (&sx)[XFRAGS],
                                         const int (&sw)[WFRAGS], AccFrag& acc) {
  v8i xf[XFRAGS], wf[WFRAGS];
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) xf[b] = read_frag(slot, xoff[b] ^ (ODD ? 64 : 0));
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) wf[a] = read_frag(slot, woff[a] ^ (ODD ? 64 : 0));
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a)
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b)
      acc.v[a][b] = ODD ? __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[a], xf[b], acc.v[a][b], 0, 0, 2, sw[a], 2, sx[b])
                        : __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[a], xf[b], acc.v[a][b], 0, 0, 0, sw[a], 0, sx[b]);
}

template <int DEPTH>
__device__ __forceinline__ void mainloop(const MokGemmResidue& g, const MokGemmTask& t, AccFrag& acc) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int r32 = lane & 31;
  const int half = lane >> 5;
  const bool gate_up = t.op == MOK_GEMM_FWD_ROUTED_GATE_UP;
  const MokMxView& act = gate_up ? g.x : g.hidden;
  const int K = act.k;
  const int nslots = (K + K_SLOT - 1) / K_SLOT;
  unsigned char* ring = pipelink_smem + pipelink_mok_gemm_arena();

  // ---- loader addresses (fixed for the tile) ---------------------------------------
  // lane -> (row lane/8 of an 8-row group, LDS position lane%8); it fetches the chunk that
  // belongs at that position
  Loader ld;
  {
    const int lrow = lane >> 3;
    const int pos = lane & 7;
    ld.chunk_byte = 16 * (pos ^ swizzle(lrow));
    static_assert(X_GROUPS % 2 == 0 && W_GROUPS % 2 == 0, "a wave's first group must start at a multiple of 16 rows");
#pragma unroll
    for (int j = 0; j < X_GROUPS; ++j) {
      const int trow = (wave * X_GROUPS + j) * 8 + lrow;  // tile-local routed row
      int row = t.row_begin + trow;
      row = row < t.row_end ? row : t.row_end - 1;
      const int src = (gate_up && g.row_token) ? g.row_token[row] : row;
      ld.xsrc[j] = (uint32_t)src * (uint32_t)act.ld_q + 16 * (pos ^ swizzle(trow));
    }
    ld.xbase = act.q;
    ld.xdst = wave * X_GROUPS * 1024;
    const MokMxView& wv = gate_up ? (wave < WAVES / 2 ? g.w_gate : g.w_up) : g.w_down;
#pragma unroll
    for (int j = 0; j < W_GROUPS; ++j) {
      const int wl = (wave * W_GROUPS + j) * 8 + lrow;  // tile-local weight row
      int col = t.col_begin + (gate_up ? (wl & (TILE_W / 2 - 1)) : wl);
      col = col < wv.rows ? col : wv.rows - 1;
      ld.wsrc[j] = (uint32_t)col * (uint32_t)wv.ld_q + 16 * (pos ^ swizzle(wl));
    }
    ld.wbase = wv.q + (int64_t)t.expert * wv.expert_pitch_q;
    ld.wdst = SLOT_X_BYTES + wave * W_GROUPS * 1024;
    // scales: thread tid < 256 fetches routed row tid's dword, the others weight row tid - 256
    if (tid < TILE_X) {
      int row = t.row_begin + tid;
      row = row < t.row_end ? row : t.row_end - 1;
      const int src = (gate_up && g.row_token) ? g.row_token[row] : row;
      ld.scbase = act.sc;
      ld.scsrc = (uint32_t)src * (uint32_t)act.ld_sc;
    } else {
      const int wl = tid - TILE_X;
      const MokMxView& sv = gate_up ? (wl < TILE_W / 2 ? g.w_gate : g.w_up) : g.w_down;
      int col = t.col_begin + (gate_up ? (wl & (TILE_W / 2 - 1)) : wl);
      col = col < sv.rows ? col : sv.rows - 1;
      ld.scbase = sv.sc + (int64_t)t.expert * sv.expert_pitch_sc;
      ld.scsrc = (uint32_t)col * (uint32_t)sv.ld_sc;
    }
    ld.scdst = SLOT_X_BYTES + SLOT_W_BYTES + wave * 256;
  }

  // ---- per-fragment LDS read offsets (step 0, first block) ---------------------------
  int xoff[XFRAGS], woff[WFRAGS], xscoff[XFRAGS], wscoff[WFRAGS];
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) {
    const int row = xrow0(wave, b) + r32;
    xoff[b] = row * K_SLOT + 16 * (half ^ swizzle(row));
    xscoff[b] = SLOT_X_BYTES + SLOT_W_BYTES + row * 4;
  }
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) {
    const int wl = wrow0(wave, a) + r32;
    woff[a] = SLOT_X_BYTES + wl * K_SLOT + 16 * (half ^ swizzle(wl));
    wscoff[a] = SLOT_X_BYTES + SLOT_W_BYTES + TILE_X * 4 + wl * 4;
  }

#pragma unroll
  for (int a = 0; a < WFRAGS; ++a)
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc.v[a][b][r] = 0.0f;

  // ---- prologue: fill depth-1 slots ---------------------------------------------------
#pragma unroll
  for (int s = 0; s < DEPTH - 1; ++s)
    if (s < nslots) issue_slot(ld, ring + s * SLOT_BYTES, s * K_SLOT, K - s * K_SLOT);

  int cur = 0;           // slot the next iteration consumes
  int fill = DEPTH - 1;  // slot the next issued load fills
  for (int i = 0; i < nslots; ++i) {
    // loads younger than slot i's: the slots i+1 .. i+DEPTH-2
    if (i + DEPTH - 2 < nslots)
      wait_vmcnt<(DEPTH - 2) * LOADS_PER_SLOT>();
    else
      wait_vmcnt<0>();
    wg_barrier();  // slot i has landed for every wave; everyone is done reading slot i-1
    if (i + DEPTH - 1 < nslots)
      issue_slot(ld, ring + fill * SLOT_BYTES, (i + DEPTH - 1) * K_SLOT, K - (i + DEPTH - 1) * K_SLOT);
    fill = fill + 1 == DEPTH ? 0 : fill + 1;
    const unsigned char* slot = ring + cur * SLOT_BYTES;
    cur = cur + 1 == DEPTH ? 0 : cur + 1;

    // block scales of the slot: lanes of the upper half use blocks 1 and 3, shifted down
    // into bytes 0 and 2 where the MFMA's op_sel picks them
    int sx[XFRAGS], sw[WFRAGS];
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b) sx[b] = (int)(*reinterpret_cast<const uint32_t*>(slot + xscoff[b]) >> (8 * half));
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) sw[a] = (int)(*reinterpret_cast<const uint32_t*>(slot + wscoff[a]) >> (8 * half));
    mma_step<false>(slot, xoff, woff, sx, sw, acc);
    if (K - i * K_SLOT > 64) mma_step<true>(slot, xoff, woff, sx, sw, acc);
  }
  wg_barrier();  // ring free for the next tile
}

__device__ __forceinline__ void store_down(const MokGemmResidue& g, const MokGemmTask& t, const AccFrag& acc) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) {
    const int row = t.row_begin + xrow0(wave, b) + (lane & 31);
    if (row >= t.row_end) continue;
    uint16_t* yrow = g.y + (int64_t)row * g.ld_y;
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = t.col_begin + wrow0(wave, a) + 8 * q + 4 * (lane >> 5);
        if (col >= g.w_down.rows) continue;  // columns come in groups of 4; extents are multiples of 32
        uint32_t p0 = __float_as_uint(bf16_round(acc.v[a][b][4 * q + 0])) >> 16;
        uint32_t p1 = __float_as_uint(bf16_round(acc.v[a][b][4 * q + 1])) & 0xFFFF0000u;
        uint32_t p2 = __float_as_uint(bf16_round(acc.v[a][b][4 * q + 2])) >> 16;
        uint32_t p3 = __float_as_uint(bf16_round(acc.v[a][b][4 * q + 3])) & 0xFFFF0000u;
        uint2 pk;
        pk.x = p0 | p1;
        pk.y = p2 | p3;
        *reinterpret_cast<uint2*>(yrow + col) = pk;
      }
    }
  }
}

}  // namespace mok_gemm_owner

extern "C" __device__ void mok_gemm_init(const void* view) { (void)view; }

// Runs the mainloop of one tile.  For the gate/up op the fp32 accumulator is left in *acc
// for the activation owner; for the down op it is rounded to bf16 and stored here.
extern "C" __device__ void mok_gemm_fwd(const void* view, const MokGemmTask* task, const MokCounters* counters,
                                        uint32_t* phase, mok::AccFrag* acc) {
  (void)counters;
  (void)phase;
  const auto& g = *static_cast<const MokGemmResidue*>(static_cast<const pipelink_host_view*>(view)->residue);
  if (pipelink_mok_gemm_depth() == 2)
    mok_gemm_owner::mainloop<2>(g, *task, *acc);
  else
    mok_gemm_owner::mainloop<3>(g, *task, *acc);  // needs 3 x 66 KB: beyond one CU's LDS at this tile size
  if (task->op == MOK_GEMM_FWD_ROUTED_DOWN) mok_gemm_owner::store_down(g, *task, *acc);
}
#else  // PIPELINK_EMIT: host-evaluated annotations only
#include "../include/mok_abi.h"
#endif

PL_STAGE("mok.gemm", "0.1.0");
PL_PARAMS(MokGemmResidue);
PL_TOPOLOGY(true, "static");
PL_VARIANT(0, {{"pipelink_mok_precision", 1}});  // MXFP8 (campaigns/mok/port/include/mok_abi.h: MOK_PRECISION_MXFP8)
PL_EXPORT(mok_gemm_init, mok_gemm_init, "extern \"C\" __device__ void mok_gemm_init(const void* view);");
PL_EXPORT(mok_gemm_fwd, mok_gemm_fwd,
          "extern \"C\" __device__ void mok_gemm_fwd(const void* view, const MokGemmTask* task, "
          "const MokCounters* counters, uint32_t* phase, mok::AccFrag* acc);");
PL_SERVE(gemm_init, "mok_gemm_init");
PL_SERVE(gemm_fwd, "mok_gemm_fwd");
// ring of `depth` slots: 256 x 128 B of routed rows, 256 x 128 B of weight rows, 2 KB of scales
PL_CLAIM_RING("pipelink_mok_gemm_arena", "smem", 0, "pipelink_mok_gemm_depth", 67584, 1024, "kernel");
PL_USES("pipelink_mok_gemm_depth");
PL_USES("pipelink_mok_gemm_arena");
PL_FACT("mok.gemm.TILE_X", 256);
PL_FACT("mok.gemm.TILE_W", 256);
PL_FACT("mok.gemm.K_SLOT", 128);
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
