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
// Ring: `depth` LDS slots of 65 KB.  A slot holds 128 contraction bytes of 256 routed rows
// and of 256 weight rows, row-major (one 128-byte cache line per row), followed by one
// dword of block scales (4 x e8m0) per weight row (weight scales are stored slot-major, so a
// tile's 1 KB of them is one contiguous load).  The routed rows' scales are row-major in HBM
// (rows are gathered); every fourth slot 16 bytes per row -- four slots' worth -- go to a
// small double buffer behind the ring.  One global_load_lds_dwordx4 moves 8 rows:
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
constexpr int LOADS_PER_SLOT = X_GROUPS + W_GROUPS + 2;  // upper bound: + weight scales + routed-row scales

// Addresses are a wave-uniform base (kept in scalar registers) plus a 32-bit lane offset: one
// operand of one expert is far below 4 GiB, and 8 + 1 offsets cost half the vector registers
// of 9 pointers.
struct Loader {
  const uint8_t* xbase;           // activations (all rows)
  const uint8_t* wbase;           // this expert's weight matrix (gate or up or down, by wave)
  const uint8_t* xscbase;         // routed rows' scales, row-major
  const uint8_t* wscbase;         // this lane's 16 bytes (4 rows) of the tile's weight scales in slot 0
  uint32_t wsc_slot_pitch;        // bytes between two slots of the weight scales
  uint32_t xscsrc;                // this thread's routed row in the scale matrix (threads 0..255)
  uint32_t xsrc[X_GROUPS];        // this lane's 16 bytes of its row in each group, at k = 0
  uint32_t wsrc[W_GROUPS];
  int chunk_byte;                 // byte offset inside the 128-byte line this lane fetches in even groups
  int xdst, wdst;                 // slot-relative LDS byte offsets of the wave's first group
};

__device__ __forceinline__ int swizzle(int row) { return (row >> 1) & 7; }

// Issue one slot.  k_left = contraction bytes from this slot's start to the end of the row:
// the last slot of a K that is not a multiple of 128 only fetches the chunks that exist.
__device__ __forceinline__ void issue_slot(const Loader& ld, unsigned char* slot, unsigned char* xscale, int kbyte,
                                           int k_left) {
  // group j starts at tile row 8 * (4 * wave + j): odd groups flip bit 2 of the swizzle, so
  // the lane's chunk there is the even-group chunk with bit 2 (64 bytes) flipped
#pragma unroll
  for (int j = 0; j < X_GROUPS; ++j)
    if ((ld.chunk_byte ^ ((j & 1) << 6)) < k_left) load16_to_lds(ld.xbase + kbyte + ld.xsrc[j], slot + ld.xdst + j * 1024);
#pragma unroll
  for (int j = 0; j < W_GROUPS; ++j)
    if ((ld.chunk_byte ^ ((j & 1) << 6)) < k_left) load16_to_lds(ld.wbase + kbyte + ld.wsrc[j], slot + ld.wdst + j * 1024);
  const int wave = threadIdx.x >> 6;
  const int s = kbyte >> 7;  // slot index
  // wave 4: the tile's weight scales of this slot, 4 rows per lane
  if (wave == 4) load16_to_lds(ld.wscbase + (size_t)s * ld.wsc_slot_pitch, slot + SLOT_X_BYTES + SLOT_W_BYTES);
  // waves 0-3, every fourth slot: 16 scale bytes of each routed row (this slot and the next three)
  if (wave < 4 && (s & 3) == 0) load16_to_lds(ld.xscbase + (kbyte >> 5) + ld.xscsrc, xscale + ((s >> 2) & 1) * (TILE_X * 16) + wave * 1024);
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
  unsigned char* xscale = ring + DEPTH * SLOT_BYTES;  // routed-row scale double buffer behind the ring

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
    // routed-row scales: thread tid < 256 fetches row tid's 16-byte piece
    {
      int row = t.row_begin + (tid & (TILE_X - 1));
      row = row < t.row_end ? row : t.row_end - 1;
      const int src = (gate_up && g.row_token) ? g.row_token[row] : row;
      ld.xscbase = act.sc;
      ld.xscsrc = (uint32_t)src * (uint32_t)act.ld_sc;
    }
    // weight scales, slot-major [slot][row][4]: lane l of one wave fetches tile rows 4l .. 4l+3
    {
      const int wl = 4 * lane;
      const MokMxView& sv = gate_up ? (wl < TILE_W / 2 ? g.w_gate : g.w_up) : g.w_down;
      int col = t.col_begin + (gate_up ? (wl & (TILE_W / 2 - 1)) : wl);
      col = col <= sv.rows - 4 ? col : sv.rows - 4;  // row counts are multiples of 32
      ld.wscbase = sv.sc + (int64_t)t.expert * sv.expert_pitch_sc + (int64_t)col * 4;
      ld.wsc_slot_pitch = (uint32_t)sv.rows * 4u;
    }
  }

  // ---- per-fragment LDS read offsets (step 0, first block) ---------------------------
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
    woff[a] = SLOT_X_BYTES + wl * K_SLOT + 16 * (half ^ swizzle(wl));
    wscoff[a] = SLOT_X_BYTES + SLOT_W_BYTES + wl * 4;
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
    if (s < nslots) issue_slot(ld, ring + s * SLOT_BYTES, xscale, s * K_SLOT, K - s * K_SLOT);

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
      issue_slot(ld, ring + fill * SLOT_BYTES, xscale, (i + DEPTH - 1) * K_SLOT, K - (i + DEPTH - 1) * K_SLOT);
    fill = fill + 1 == DEPTH ? 0 : fill + 1;
    const unsigned char* slot = ring + cur * SLOT_BYTES;
    cur = cur + 1 == DEPTH ? 0 : cur + 1;

    // block scales of the slot: lanes of the upper half use blocks 1 and 3, shifted down
    // into bytes 0 and 2 where the MFMA's op_sel picks them
    int sx[XFRAGS], sw[WFRAGS];
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b)
      sx[b] = (int)(*reinterpret_cast<const uint32_t*>(xscale + ((i >> 2) & 1) * (TILE_X * 16) + xscoff[b] + 4 * (i & 3)) >> (8 * half));
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) sw[a] = (int)(*reinterpret_cast<const uint32_t*>(slot + wscoff[a]) >> (8 * half));
    mma_step<false>(slot, xoff, woff, sx, sw, acc);
    if (K - i * K_SLOT > 64) mma_step<true>(slot, xoff, woff, sx, sw, acc);
  }
  wg_barrier();  // ring free for the next tile
}

// bf16 epilogue of the down op.  The accumulator is transposed through the (now idle) ring so
// that the global stores are 16 bytes per lane and 512 contiguous bytes per routed row.
constexpr int Y_PITCH = TILE_W * 2 + 16;  // bytes per staged row: 256 bf16 + pad against bank conflicts
static_assert(TILE_X * Y_PITCH <= 2 * SLOT_BYTES + XSCALE_BYTES, "staging tile must fit the two-slot ring");

typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2));  // v_cvt_pk_bf16_f32, nearest even
}

__device__ __forceinline__ void store_down(const MokGemmResidue& g, const MokGemmTask& t, const AccFrag& acc) {
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  unsigned char* stage = pipelink_smem + pipelink_mok_gemm_arena();
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) {
    unsigned char* rowp = stage + (xrow0(wave, b) + (lane & 31)) * Y_PITCH;
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = wrow0(wave, a) + 8 * q + 4 * (lane >> 5);
        uint2 pk;
        pk.x = pack_bf16x2(acc.v[a][b][4 * q + 0], acc.v[a][b][4 * q + 1]);
        pk.y = pack_bf16x2(acc.v[a][b][4 * q + 2], acc.v[a][b][4 * q + 3]);
        *reinterpret_cast<uint2*>(rowp + col * 2) = pk;
      }
    }
  }
  __syncthreads();
  const int chunk = lane & 31;                              // 8 columns = 16 bytes
  const bool col_ok = t.col_begin + chunk * 8 < g.w_down.rows;  // column extents are multiples of 32
#pragma unroll 4
  for (int it = 0; it < TILE_X / 16; ++it) {
    const int trow = wave * (TILE_X / 8) + it * 2 + (lane >> 5);
    const int row = t.row_begin + trow;
    if (row < t.row_end && col_ok) {
      const uint4 v = *reinterpret_cast<const uint4*>(stage + trow * Y_PITCH + chunk * 16);
      *reinterpret_cast<uint4*>(g.y + (int64_t)row * g.ld_y + t.col_begin + chunk * 8) = v;
    }
  }
  __syncthreads();  // the ring is reused by the next tile's loads
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
// ring of `depth` slots: 256 x 128 B of routed rows, 256 x 128 B of weight rows, 1 KB of weight scales
// + 8 KB behind the ring: double buffer of the routed rows' scales
PL_CLAIM_RING("pipelink_mok_gemm_arena", "smem", 8192, "pipelink_mok_gemm_depth", 66560, 1024, "phase:instr_gemm");
PL_USES("pipelink_mok_gemm_depth");
PL_USES("pipelink_mok_gemm_arena");
PL_FACT("mok.gemm.TILE_X", 256);
PL_FACT("mok.gemm.TILE_W", 256);
PL_FACT("mok.gemm.K_SLOT", 128);
PL_PRELUDE("../include/mok_abi.h");
PL_PRELUDE("../include/mok_device.hpp");
PL_EMIT_MAIN()
