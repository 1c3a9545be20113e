// Package oe.mma.full: the matrix side of the one-epilogue example at the tile the accumulation registers allow,
// 256 x 256 per workgroup, 128 x 128 per wave in 256 AGPRs.  A wave then needs every register of its SIMD lane, so
// there is no room for loader waves beside it: the four waves bring their own operands (LDS-DMA loads placed between
// their MFMAs), and the package is loader and matrix role in one.  Per 32 contraction elements a workgroup moves
// 32 KB through L2 and LDS for 4.2 MFLOP: half the bytes per flop of the 256 x 128 tile, a quarter of the 128 x 128 one.
//
// Operand roles are swapped with respect to C = A . B: the B^T rows (output columns) feed the MFMA's first operand and
// the A rows its second, so the accumulator a wave hands over is the transpose of its share of C -- tensor rows are
// output columns, tensor columns output rows -- and one lane holds four consecutive output columns of one output row,
// which is what a row-major bf16 store wants.  The products and their order of summation are those of the other
// matrix packages (16 contraction elements per MFMA, ascending), so the result has the same bits.
//
// LDS: two rings of five 16 KB buffers (all 160 KB), one for the A rows and one for the B^T rows.  A buffer holds 32
// contraction elements (64 bytes, a "slot") of 256 rows, row-major; one buffer_load_dwordx4 ... lds moves 16 rows,
// four lanes covering the 64 bytes of a row; the four 16-byte chunks of a row are stored at position
// chunk ^ ((row / 4) % 4), which makes a fragment read (16 lanes = 16 consecutive rows, one chunk each) touch 16
// different 16-byte bank groups.  Both matrices are row-major with the contraction innermost, so a row's two
// consecutive slots are the two halves of one 128-byte line: they are asked for back to back (a pair costs the memory
// system what one full-line request costs) and land in two buffers.
//
// Schedule: step t multiplies slot t out of registers (32 MFMAs per wave) while the wave reads slot t + 1 from LDS into
// a second register set and issues its share of a pair four slots ahead; one s_barrier per step says that slot t + 1
// has landed for every wave and that every wave holds slot t in registers, i.e. slot t's buffers are free.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <type_traits>
#include <utility>
#include <hip/hip_runtime.h>
#include "include/oe_abi.h"

extern "C" __device__ int pipelink_oe_full_ring();  // byte offset of the two rings in dynamic LDS
extern "C" __device__ void pipelink_call_epilogue(const void* view, const OeTile* tile, const void* source);

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace oe_full {
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __amdgpu_buffer_rsrc_t rsrc_t;
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int TILE = OE_FULL_TILE;     // rows of either operand per workgroup
constexpr int SLOT = 64;               // contraction bytes per buffer row
constexpr int BUF = TILE * SLOT;       // 16 KB
constexpr int NB = OE_FULL_BUFFERS;    // buffers per ring
constexpr int GROUPS = TILE / 16 / 4;  // 16-row load groups per wave and operand
constexpr int FR = 4;                  // 32-row fragments per wave and operand

__device__ __forceinline__ int swizzle(int row) { return (row >> 2) & 3; }
__device__ __forceinline__ void wg_barrier() {  // no fence: the explicit waits in front order the LDS traffic
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}
// at most N global loads outstanding, every LDS read returned
template <int N>
__device__ __forceinline__ void wait_loads_and_reads() {
  static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit field");
  __builtin_amdgcn_s_waitcnt(0x0070 | (N & 0xF) | ((N >> 4) << 14));
}

struct Loader {
  rsrc_t a, b;
  uint32_t asrc[GROUPS], bsrc[GROUPS];  // this lane's 16 bytes of its row in each group, at contraction byte 0
  unsigned char* ring_a;                // first A buffer + this wave's first group
  unsigned char* ring_b;
};
// both halves of the 128-byte line that starts at slot `s` (even) of row group G: into buffers b0 and b1
template <int G>
__device__ __forceinline__ void issue_group(const Loader& ld, int s, int b0, int b1) {
  const int k = s * SLOT;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(ld.a, (lds_ptr)(ld.ring_a + b0 * BUF + G * 1024), 16, (int)ld.asrc[G], k, 0, 0);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(ld.a, (lds_ptr)(ld.ring_a + b1 * BUF + G * 1024), 16, (int)ld.asrc[G], k + SLOT, 0, 0);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(ld.b, (lds_ptr)(ld.ring_b + b0 * BUF + G * 1024), 16, (int)ld.bsrc[G], k, 0, 0);
  __builtin_amdgcn_raw_ptr_buffer_load_lds(ld.b, (lds_ptr)(ld.ring_b + b1 * BUF + G * 1024), 16, (int)ld.bsrc[G], k + SLOT, 0, 0);
}
// one of the eight loads of a step: L = 0..7 -> group G0 + L / 4, then A first half, A second half, B first, B second
template <int G0, int L>
__device__ __forceinline__ void issue_one(const Loader& ld, int s, int b0, int b1) {
  constexpr int G = G0 + L / 4, OPERAND = (L / 2) % 2, HALF = L % 2;
  __builtin_amdgcn_raw_ptr_buffer_load_lds(OPERAND ? ld.b : ld.a, (lds_ptr)((OPERAND ? ld.ring_b : ld.ring_a) + (HALF ? b1 : b0) * BUF + G * 1024), 16,
                                           (int)(OPERAND ? ld.bsrc[G] : ld.asrc[G]), s * SLOT + HALF * SLOT, 0, 0);
}

// a slot's operands of one wave: per 32-row fragment the lane's 16 bytes of the slot's first 16 elements and of its second
struct Operands {
  v4i a[2][FR], b[2][FR];
};

__device__ __forceinline__ int next_buffer(int b) { return b + 1 == NB ? 0 : b + 1; }
__device__ __forceinline__ int buffer_plus(int b, int by) {  // (b + by) mod NB for 0 <= b < NB, 0 <= by <= NB
  const int c = b + by;
  return c >= NB ? c - NB : c;
}
}  // namespace oe_full

extern "C" __device__ void oe_mma_full_role_mma(const void* params, unsigned variant) {
  (void)variant;
  using namespace oe_full;
  const OeFullParams& p = *static_cast<const OeFullParams*>(params);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
  const int tiles_n = p.n / TILE;
  const int tile_m = (int)blockIdx.x / tiles_n, tile_n = (int)blockIdx.x % tiles_n;
  unsigned char* ring = pipelink_smem + pipelink_oe_full_ring();
  const uint32_t pitch = (uint32_t)p.k * 2u;

  Loader ld;
  ld.a = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.a), 0, (int)((uint32_t)p.m * pitch), 0x00020000);
  ld.b = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t*>(p.bt), 0, (int)((uint32_t)p.n * pitch), 0x00020000);
  {
    const int lrow = lane >> 2, chunk = 16 * ((lane & 3) ^ swizzle(lrow));
#pragma unroll
    for (int g = 0; g < GROUPS; ++g) {
      const int row = (wave * GROUPS + g) * 16 + lrow;  // tile-local; groups start at multiples of 16, so swizzle(row) = swizzle(lrow)
      ld.asrc[g] = (uint32_t)(tile_m * TILE + row) * pitch + chunk;
      ld.bsrc[g] = (uint32_t)(tile_n * TILE + row) * pitch + chunk;
    }
    ld.ring_a = ring + wave * GROUPS * 1024;
    ld.ring_b = ring + NB * BUF + wave * GROUPS * 1024;
  }
  // fragment reads: the lane's row of fragment f, chunk lane / 32 (first 16 elements) and that + 2 (second 16)
  const int wn = wave & 1, wm = wave >> 1, r32 = lane & 31, half = lane >> 5;
  int aoff[FR], boff[FR];
#pragma unroll
  for (int f = 0; f < FR; ++f) {
    const int arow = 128 * wm + 32 * f + r32, brow = 128 * wn + 32 * f + r32;
    aoff[f] = arow * SLOT + 16 * (half ^ swizzle(arow));
    boff[f] = NB * BUF + brow * SLOT + 16 * (half ^ swizzle(brow));
  }
  // acc[i][j]: B^T-row fragment i (output columns) x A-row fragment j (output rows)
  v16f acc[FR][FR];
#pragma unroll
  for (int i = 0; i < FR; ++i)
#pragma unroll
    for (int j = 0; j < FR; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

  const int n = p.k / 32;  // slots; even and at least 8 (the host checks)
  // prologue: the pairs (0, 1) and (2, 3), whole
  issue_group<0>(ld, 0, 0, 1); issue_group<1>(ld, 0, 0, 1); issue_group<2>(ld, 0, 0, 1); issue_group<3>(ld, 0, 0, 1);
  issue_group<0>(ld, 2, 2, 3); issue_group<1>(ld, 2, 2, 3); issue_group<2>(ld, 2, 2, 3); issue_group<3>(ld, 2, 2, 3);
  wait_loads_and_reads<16>();  // pair (0, 1) has landed
  wg_barrier();

  Operands even, odd;
  auto read_one = [&](Operands& o, int buf, auto K_) {  // K = 0..15: first halves of a0..a3, b0..b3, then second halves
    constexpr int K = decltype(K_)::value;
    constexpr int H = K / 8, F = K % 4;
    const unsigned char* base = ring + buf * BUF;
    if constexpr ((K / 4) % 2 == 0) o.a[H][F] = *reinterpret_cast<const v4i*>(base + (aoff[F] ^ (32 * H)));
    else o.b[H][F] = *reinterpret_cast<const v4i*>(base + (boff[F] ^ (32 * H)));
  };
  auto read_all = [&](Operands& o, int buf) {
    read_one(o, buf, std::integral_constant<int, 0>{}); read_one(o, buf, std::integral_constant<int, 1>{});
    read_one(o, buf, std::integral_constant<int, 2>{}); read_one(o, buf, std::integral_constant<int, 3>{});
    read_one(o, buf, std::integral_constant<int, 4>{}); read_one(o, buf, std::integral_constant<int, 5>{});
    read_one(o, buf, std::integral_constant<int, 6>{}); read_one(o, buf, std::integral_constant<int, 7>{});
    read_one(o, buf, std::integral_constant<int, 8>{}); read_one(o, buf, std::integral_constant<int, 9>{});
    read_one(o, buf, std::integral_constant<int, 10>{}); read_one(o, buf, std::integral_constant<int, 11>{});
    read_one(o, buf, std::integral_constant<int, 12>{}); read_one(o, buf, std::integral_constant<int, 13>{});
    read_one(o, buf, std::integral_constant<int, 14>{}); read_one(o, buf, std::integral_constant<int, 15>{});
  };
  auto mfma = [&](const Operands& o, int h, int i, int j) {
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, o.b[h][i]), __builtin_bit_cast(v8bf, o.a[h][j]), acc[i][j], 0, 0, 0);
  };
  read_all(even, 0);

  // One step: the 32 MFMAs of slot t (16 element 0-15 products, then 16 element 16-31 products: 16 MFMAs between two
  // on one accumulator), with the wait and the barrier behind the fourth, the 16 reads of slot t + 1 and the step's 8
  // loads spread between the MFMAs behind that.  WAIT: loads that may still be in flight behind slot t + 1's.
  // ISSUE: 0 none, 1 groups 0-1 of the pair that starts at slot t + 4 (even steps), 2 groups 2-3 of the pair that
  // starts at slot t + 3 (odd steps).  `buf` is slot t's buffer.
  auto step = [&](auto WAIT_, auto ISSUE_, auto READ_, const Operands& cur, Operands& next, int t, int buf) {
    constexpr int WAIT = decltype(WAIT_)::value, ISSUE = decltype(ISSUE_)::value;
    constexpr bool READ = decltype(READ_)::value;
    const int nbuf = next_buffer(buf);
    // even step: slots t + 4, t + 5 go where slots t - 1 and t were; odd step: slots t + 3, t + 4 where t - 2 and t - 1 were
    const int b0 = ISSUE == 1 ? buffer_plus(buf, NB - 1) : buffer_plus(buf, NB - 2);
    const int b1 = ISSUE == 1 ? buf : buffer_plus(buf, NB - 1);
    const int s = ISSUE == 1 ? t + 4 : t + 3;
    auto place = [&](auto I_) {
      constexpr int I = decltype(I_)::value;
      mfma(cur, I / 16, (I % 16) / FR, I % FR);
      __builtin_amdgcn_sched_barrier(0);
      if constexpr (I == 3 && READ) {
        wait_loads_and_reads<WAIT>();
        wg_barrier();
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (READ && I >= 4 && I < 20) read_one(next, nbuf, std::integral_constant<int, I - 4>{});
      if constexpr (ISSUE != 0 && I >= 6 && I < 30 && (I - 6) % 3 == 0) issue_one<ISSUE == 1 ? 0 : 2, (I - 6) / 3>(ld, s, b0, b1);
      __builtin_amdgcn_sched_barrier(0);
    };
    __builtin_amdgcn_sched_barrier(0);
    place(std::integral_constant<int, 0>{}); place(std::integral_constant<int, 1>{}); place(std::integral_constant<int, 2>{});
    place(std::integral_constant<int, 3>{}); place(std::integral_constant<int, 4>{}); place(std::integral_constant<int, 5>{});
    place(std::integral_constant<int, 6>{}); place(std::integral_constant<int, 7>{}); place(std::integral_constant<int, 8>{});
    place(std::integral_constant<int, 9>{}); place(std::integral_constant<int, 10>{}); place(std::integral_constant<int, 11>{});
    place(std::integral_constant<int, 12>{}); place(std::integral_constant<int, 13>{}); place(std::integral_constant<int, 14>{});
    place(std::integral_constant<int, 15>{}); place(std::integral_constant<int, 16>{}); place(std::integral_constant<int, 17>{});
    place(std::integral_constant<int, 18>{}); place(std::integral_constant<int, 19>{}); place(std::integral_constant<int, 20>{});
    place(std::integral_constant<int, 21>{}); place(std::integral_constant<int, 22>{}); place(std::integral_constant<int, 23>{});
    place(std::integral_constant<int, 24>{}); place(std::integral_constant<int, 25>{}); place(std::integral_constant<int, 26>{});
    place(std::integral_constant<int, 27>{}); place(std::integral_constant<int, 28>{}); place(std::integral_constant<int, 29>{});
    place(std::integral_constant<int, 30>{}); place(std::integral_constant<int, 31>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  using W0 = std::integral_constant<int, 0>;
  using W8 = std::integral_constant<int, 8>;
  using W16 = std::integral_constant<int, 16>;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  // Slot t + 1's last loads were issued in step t - 3 (t even: it is the second slot of its pair) or t - 2 (t odd), so
  // two steps' loads (16) or one step's (8) may still be outstanding behind them.
  int t = 0, buf = 0;
  for (; t + 6 <= n; t += 2) {  // both steps still issue: the last pair (n - 2, n - 1) is issued in steps n - 6, n - 5
    step(W16{}, I1{}, std::true_type{}, even, odd, t, buf);
    buf = next_buffer(buf);
    step(W8{}, I2{}, std::true_type{}, odd, even, t + 1, buf);
    buf = next_buffer(buf);
  }
  // t = n - 4: nothing left to issue
  step(W16{}, I0{}, std::true_type{}, even, odd, t, buf);
  buf = next_buffer(buf);
  step(W0{}, I0{}, std::true_type{}, odd, even, t + 1, buf);
  buf = next_buffer(buf);
  step(W0{}, I0{}, std::true_type{}, even, odd, t + 2, buf);
  buf = next_buffer(buf);
  step(W0{}, I0{}, std::false_type{}, odd, even, t + 3, buf);

  // the frame handed over: 16 floats per fragment and lane in fragment order, pinned in the accumulation registers
  const OeTile tile{tile_n * TILE + 128 * wn, tile_m * TILE + 128 * wm};  // the transpose's first row (output column), first column (output row)
  float frame[FR * FR * 16];
#pragma unroll
  for (int i = 0; i < FR; ++i)
#pragma unroll
    for (int j = 0; j < FR; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float v = acc[i][j][r];
        asm volatile("" : "+a"(v));
        frame[(i * FR + j) * 16 + r] = v;
      }
  const pipelink_host_view view{params, nullptr};
  pipelink_call_epilogue(&view, &tile, frame);
}
#else
#include "include/oe_abi.h"
#endif

PL_STAGE("oe.mma.full", "0.1.0");
PL_PARAMS(OeFullParams);
PL_ROLE(mma, oe_mma_full_role_mma, 4);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_CALL(epilogue, "oe_epilogue_full_store",
        "extern \"C\" __device__ void pipelink_call_epilogue(const void* view, const OeTile* tile, const void* source);");
// the wave's share of C, transposed: 128 output columns x 128 output rows
PL_EXPORT_TENSOR(acc, "gemm_accumulator_transposed", "f32", 128, 128, "agpr", "mfma32x32c", 0);
PL_CLAIM("pipelink_oe_full_ring", "smem", 2 * OE_FULL_BUFFERS * OE_FULL_TILE * 64, 1024, "kernel");
PL_USES("pipelink_oe_full_ring");
PL_PRELUDE("include/oe_abi.h");
PL_EMIT_MAIN()
