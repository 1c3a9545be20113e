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
// Ring: `depth` LDS stages of 24 KB, each holding 64 contraction bytes of 128 routed rows
// and 256 weight rows in [16-byte chunk][row] order: a wave's global_load_lds of one chunk
// of 64 consecutive rows lands contiguously, and a fragment read (32 lanes, 16 bytes each,
// consecutive rows) is contiguous too, so neither side has bank conflicts.  The depth is a
// link-time handle; the ring offset inside the workgroup's dynamic LDS is another.
#include "../include/mok_device.hpp"

extern "C" __device__ int pipelink_mok_gemm_depth();  // ring stages (2..6), bound at link time
extern "C" __device__ int pipelink_mok_gemm_arena();  // byte offset of the ring in dynamic LDS

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mok_gemm_owner {
using namespace mok;

constexpr int LOADS_PER_STEP = STAGE_BYTES / (THREADS * 16);  // 6 direct-to-LDS loads per lane

struct Loader {
  const uint8_t* xsrc;  // this lane's routed row, at this wave's first chunk
  const uint8_t* wsrc;  // this lane's weight row
  int xdst;             // stage-relative LDS byte offsets of the wave's first chunk
  int wdst;
};

__device__ __forceinline__ void issue_stage(const Loader& ld, unsigned char* stage, int kbyte) {
  // activations: 2 chunks per wave; weights: 4 chunks per wave
  load16_to_lds(ld.xsrc + kbyte, stage + ld.xdst);
  load16_to_lds(ld.xsrc + kbyte + 16, stage + ld.xdst + TILE_X * 16);
#pragma unroll
  for (int c = 0; c < 4; ++c)
    load16_to_lds(ld.wsrc + kbyte + 16 * c, stage + ld.wdst + c * TILE_W * 16);
}

// MFMA 32x32x64 f8f6f4 operand of lane (row = lane % 32, half = lane / 32): registers 0-3
// hold 16 bytes of the step's first 32-element block, registers 4-7 16 bytes of its second
// block; the scale of block 0 is taken from lanes 0-31 and that of block 1 from lanes 32-63
// (measured on gfx950 with a one-instruction probe).  So a lane reads chunk `half` and
// chunk `half + 2` of its row.
__device__ __forceinline__ v8i read_frag(const unsigned char* chunk_lo, int plane_bytes) {
  const v4i lo = *reinterpret_cast<const v4i*>(chunk_lo);
  const v4i hi = *reinterpret_cast<const v4i*>(chunk_lo + 2 * plane_bytes);
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

template <int DEPTH>
struct Ring {
  unsigned char* base;
  int slot;  // stage the next step consumes
  int fill;  // stage the next issued load fills
};

// One 64-element contraction step: wait for its stage, refill the stage freed by the
// previous step, read 6 fragments, issue 8 MFMAs.
template <int DEPTH, bool ODD>
__device__ __forceinline__ void step(const Loader& ld, Ring<DEPTH>& rs, int i, int nk, const int (&xoff)[XFRAGS],
                                     const int (&woff)[WFRAGS], const int (&sx)[XFRAGS], const int (&sw)[WFRAGS],
                                     AccFrag& acc) {
  // Loads younger than stage i's: the stages i+1 .. i+DEPTH-2 and the pair's batch of scale
  // dwords, which is issued at the top of the even step -- after stage i's loads except for
  // the odd step of a two-stage ring, whose stage is only issued inside the even step.
  constexpr int YOUNGER_SCALES = (ODD && DEPTH == 2) ? 0 : XFRAGS + WFRAGS;
  if (i + DEPTH - 2 < nk)
    wait_vmcnt<(DEPTH - 2) * LOADS_PER_STEP + YOUNGER_SCALES>();
  else
    wait_vmcnt<0>();
  wg_barrier();
  if (i + DEPTH - 1 < nk) issue_stage(ld, rs.base + rs.fill * STAGE_BYTES, (i + DEPTH - 1) * K_STEP);
  rs.fill = rs.fill + 1 == DEPTH ? 0 : rs.fill + 1;
  const unsigned char* stage = rs.base + rs.slot * STAGE_BYTES;
  rs.slot = rs.slot + 1 == DEPTH ? 0 : rs.slot + 1;
  v8i xf[XFRAGS], wf[WFRAGS];
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) xf[b] = read_frag(stage + xoff[b], TILE_X * 16);
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) wf[a] = read_frag(stage + woff[a], TILE_W * 16);
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
  const int nk = act.k / K_STEP;
  unsigned char* ring = pipelink_smem + pipelink_mok_gemm_arena();

  // ---- loader addresses (fixed for the tile) ---------------------------------------
  Loader ld;
  {
    int row = t.row_begin + (wave & 1) * 64 + lane;
    row = row < t.row_end ? row : t.row_end - 1;
    const int src = (gate_up && g.row_token) ? g.row_token[row] : row;
    ld.xsrc = act.q + (int64_t)src * act.ld_q + (wave >> 1) * 32;
    ld.xdst = (wave >> 1) * 2 * (TILE_X * 16) + (wave & 1) * 1024;
    const int wl = wave * 64 + lane;  // tile-local weight row
    const MokMxView& wv = gate_up ? (wave < 2 ? g.w_gate : g.w_up) : g.w_down;
    int col = t.col_begin + (gate_up ? (wl & (TILE_W / 2 - 1)) : wl);
    col = col < wv.rows ? col : wv.rows - 1;
    ld.wsrc = wv.q + (int64_t)t.expert * wv.expert_pitch_q + (int64_t)col * wv.ld_q;
    ld.wdst = STAGE_X_BYTES + wave * 1024;
  }

  // ---- per-fragment scale rows and LDS read offsets --------------------------------
  const uint8_t* xsc[XFRAGS];
  const uint8_t* wsc[WFRAGS];
  int xoff[XFRAGS], woff[WFRAGS];
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) {
    int row = t.row_begin + xrow0(wave, b) + r32;
    row = row < t.row_end ? row : t.row_end - 1;
    const int src = (gate_up && g.row_token) ? g.row_token[row] : row;
    xsc[b] = act.sc + (int64_t)src * act.ld_sc;
    xoff[b] = half * (TILE_X * 16) + (xrow0(wave, b) + r32) * 16;
  }
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) {
    const int wl = wrow0(wave, a) + r32;
    const MokMxView& wv = gate_up ? (a < 2 ? g.w_gate : g.w_up) : g.w_down;
    int col = t.col_begin + (gate_up ? (wl & (TILE_W / 2 - 1)) : wl);
    col = col < wv.rows ? col : wv.rows - 1;
    wsc[a] = wv.sc + (int64_t)t.expert * wv.expert_pitch_sc + (int64_t)col * wv.ld_sc;
    woff[a] = STAGE_X_BYTES + half * (TILE_W * 16) + wl * 16;
  }

#pragma unroll
  for (int a = 0; a < WFRAGS; ++a)
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc.v[a][b][r] = 0.0f;

  // ---- prologue: scales of the first pair, then depth-1 stages -----------------------
  int sx[XFRAGS], sw[WFRAGS], sx_next[XFRAGS], sw_next[WFRAGS];
  const int npairs = (nk + 1) >> 1;
#pragma unroll
  for (int b = 0; b < XFRAGS; ++b) sx[b] = (int)(*reinterpret_cast<const uint32_t*>(xsc[b]) >> (8 * half));
#pragma unroll
  for (int a = 0; a < WFRAGS; ++a) sw[a] = (int)(*reinterpret_cast<const uint32_t*>(wsc[a]) >> (8 * half));
#pragma unroll
  for (int s = 0; s < DEPTH - 1; ++s)
    if (s < nk) issue_stage(ld, ring + s * STAGE_BYTES, s * K_STEP);

  Ring<DEPTH> rs{ring, 0, DEPTH - 1};
  for (int p = 0; p < npairs; ++p) {
    // Scale bytes of the next 128-element pair: one dword per row.  Issued before this
    // pair's stage loads so that waiting for them never drains younger stage loads; the
    // last pair re-reads its own dword to keep the number of loads in flight uniform.
    const int pn = p + 1 < npairs ? p + 1 : p;
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b) sx_next[b] = (int)*reinterpret_cast<const uint32_t*>(xsc[b] + 4 * pn);
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) sw_next[a] = (int)*reinterpret_cast<const uint32_t*>(wsc[a] + 4 * pn);
    step<DEPTH, false>(ld, rs, 2 * p, nk, xoff, woff, sx, sw, acc);
    if (2 * p + 1 < nk) step<DEPTH, true>(ld, rs, 2 * p + 1, nk, xoff, woff, sx, sw, acc);
    // lanes of the upper half use blocks 1 and 3: shift them down into bytes 0 and 2
#pragma unroll
    for (int b = 0; b < XFRAGS; ++b) sx[b] = (int)((uint32_t)sx_next[b] >> (8 * half));
#pragma unroll
    for (int a = 0; a < WFRAGS; ++a) sw[a] = (int)((uint32_t)sw_next[a] >> (8 * half));
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
  switch (pipelink_mok_gemm_depth()) {
    case 2: mok_gemm_owner::mainloop<2>(g, *task, *acc); break;
    case 3: mok_gemm_owner::mainloop<3>(g, *task, *acc); break;
    case 4: mok_gemm_owner::mainloop<4>(g, *task, *acc); break;
    case 5: mok_gemm_owner::mainloop<5>(g, *task, *acc); break;
    default: mok_gemm_owner::mainloop<6>(g, *task, *acc); break;
  }
  if (task->op == MOK_GEMM_FWD_ROUTED_DOWN) mok_gemm_owner::store_down(g, *task, *acc);
}
