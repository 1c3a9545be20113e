// Package fa.core: flash-attention forward for one tile of 128 queries of one head.
//
// Orientation.  Scores are computed transposed, S^T = K . Q^T (keys are the MFMA rows, queries the
// columns), so that a lane holds ONE query (column lane % 32) and 16 of the block's 32 keys: row maxima
// and sums are in-register reductions plus one exchange between lane l and l ^ 32.  The probabilities
// are then, register for register, the B operand of O^T += V^T . P^T -- the contraction index of an MFMA
// is only a summation order, and V^T is read from LDS in the order the registers hold the keys:
//   group g of 16 keys (registers 8g .. 8g+7 of a 32-key score tile), lane half h = lane / 32:
//   elements 0-3 = keys 16g + 4h + 0..3, elements 4-7 = keys 16g + 8 + 4h + 0..3.
// K and V both go global -> LDS as stored (row-major [key][d], the 16-byte chunks of a row permuted so that the
// reads below meet no bank conflict: k_place / v_place).  K rows are the A operand of the first product as they are.  The A operand of the
// second product wants, per lane, four consecutive KEYS at one d -- a column of the V tile: that is what
// ds_read_b64_tr_b16 delivers.  In a group of 16 lanes, lane i hands in the address of 4 consecutive d
// (8 bytes) and lane j receives element j % 4 of the data of lanes j / 4, j / 4 + 4, j / 4 + 8, j / 4 + 12
// (measured with a probe); so lane i points at key kbase + i / 4, d = dbase + 4 (i % 4), and lane j gets keys
// kbase .. kbase + 3 at d = dbase + j.
//
// Two LDS buffers per operand: block i + 1 is in flight while block i is multiplied; one barrier per block.
#include <pipelink/stage.hpp>
#ifndef PIPELINK_EMIT
#include <hip/hip_runtime.h>
#include <type_traits>
#include "include/fa_abi.h"

extern "C" __device__ int pipelink_fa_kv();  // byte offset of the K / V^T buffers in dynamic LDS
extern "C" __device__ int pipelink_call_mask_key_count(const void* view, int q_first, int q_last);
extern "C" __device__ int pipelink_call_mask_key_begin(const void* view, int q_first, int q_last);
extern "C" __device__ int pipelink_call_mask_all_visible(const void* view, int q_first, int q_last, int k_first, int k_last);
extern "C" __device__ int pipelink_call_mask_visible(const void* view, int q, int k);

extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace fa_core {
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef __bf16 v4bf __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v8f __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) void* lds_ptr;

constexpr int K_BYTES = FA_K_BLOCK * FA_D * 2;     // 16 KB: [64 keys][256 bytes], the same for V
constexpr int BUF_BYTES = 2 * K_BYTES;
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s* lds_v4s;
constexpr float MASKED = -1.0e30f;
constexpr float RESCALE_SLACK = 8.0f;  // log2 units

// Where the 16-byte chunk `chunk` of a key's row stands in its 256-byte LDS row.  K is read one key per lane, 16 lanes
// = 16 consecutive keys at one chunk: the 16 rows must put that chunk in 16 different places.  V is read in columns,
// 32 lanes = 4 consecutive keys x 4 consecutive chunks: the 4 rows must put each group of 4 chunks in a different place.
__device__ __forceinline__ int k_place(int key, int chunk) { return chunk ^ (key & 15); }
__device__ __forceinline__ int v_place(int key, int chunk) { return chunk ^ (4 * (key & 3)); }

// one 64-key block of K or V -> LDS: 64 keys x 256 B; one load instruction of a wave moves 4 keys (1 KB)
template <bool IS_V>
__device__ __forceinline__ void issue_block(__amdgpu_buffer_rsrc_t src, uint32_t first_key_byte, unsigned char* dst, int wave, int lane) {
  const int kr = lane >> 4, pos = lane & 15;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int key = (wave * 4 + j) * 4 + kr;  // 0..63
    const uint32_t off = first_key_byte + (uint32_t)key * (FA_D * 2) + 16u * (uint32_t)(IS_V ? v_place(key, pos) : k_place(key, pos));
    __builtin_amdgcn_raw_ptr_buffer_load_lds(src, (lds_ptr)(dst + (wave * 4 + j) * 1024), 16, (int)off, 0, 0, 0);
  }
}
// The transposing read: in a group of 16 lanes, lane i hands in the address of 4 consecutive d of key kbase + i / 4
// and lane j receives keys kbase .. kbase + 3 at d = dbase + j.
__device__ __forceinline__ v4s read_v_piece(const unsigned char* at) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s)(const_cast<unsigned char*>(at)));
}
// A value of this lane and the one of lane ^ 32, without a trip through the LDS: after the swap the first result
// holds the lower half-wave's values in both halves, the second the upper half-wave's.
__device__ __forceinline__ float max_with_other_half(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float sum_with_other_half(float v) {
  const auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
}  // namespace fa_core

extern "C" __device__ void fa_core_role_core(const void* params, unsigned variant) {
  (void)variant;
  using namespace fa_core;
  const FaCoreParams& p = *static_cast<const FaCoreParams*>(params);
  const pipelink_host_view view{params, nullptr};
  const int tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = lane >> 5, l32 = lane & 31;
  const int q_tiles = p.seq / FA_Q_TILE;
  // Causal tiles cost in proportion to their position: the latest (longest) tiles of every head are
  // dispatched first, so that the grid does not end on a few long ones.  bh = batch * q_heads + head.
  const int heads = p.batch * p.q_heads;
  const int tile = q_tiles - 1 - (int)(blockIdx.x / heads), bh = blockIdx.x % heads;
  const int b = bh / p.q_heads, h = bh % p.q_heads, kvh = h / (p.q_heads / p.kv_heads);
  const int q0 = tile * FA_Q_TILE, qw = q0 + 32 * wave;               // the wave's first query
  const uint32_t head_bytes = (uint32_t)p.seq * FA_D * 2;
  const __amdgpu_buffer_rsrc_t kres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.k) + ((int64_t)b * p.kv_heads + kvh) * p.seq * FA_D, 0, (int)head_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t vres = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<uint16_t*>(p.v) + ((int64_t)b * p.kv_heads + kvh) * p.seq * FA_D, 0, (int)head_bytes, 0x00020000);
  unsigned char* buf = pipelink_smem + pipelink_fa_kv();

  // this lane's query row as the B operand of S^T = K . Q^T: 16 bytes per 16-element step of d
  v8bf qf[8];
  {
    const uint16_t* qrow = p.q + (((int64_t)b * p.q_heads + h) * p.seq + qw + l32) * FA_D;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) qf[kk] = __builtin_bit_cast(v8bf, *reinterpret_cast<const v4i*>(qrow + 16 * kk + 8 * half));
  }
  v16f o[4];  // O^T: [d block][16 d of the block] for this lane's query
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[db][r] = 0.0f;
  float row_max = MASKED, row_sum = 0.0f;
  bool seen = false;  // this lane's query has met a key it may see (decided on unscaled scores: the scale is the caller's)

  // the mask package says which stretch of keys the tile's queries may see at all: blocks [first_block, blocks)
  const int keys = pipelink_call_mask_key_count(&view, q0, q0 + FA_Q_TILE - 1);
  const int first_block = pipelink_call_mask_key_begin(&view, q0, q0 + FA_Q_TILE - 1) / FA_K_BLOCK;
  const int blocks = (keys + FA_K_BLOCK - 1) / FA_K_BLOCK;
  const int wave_keys = pipelink_call_mask_key_count(&view, qw, qw + 31), wave_begin = pipelink_call_mask_key_begin(&view, qw, qw + 31);
  // Schedule.  Two LDS buffers per operand: block i + 1 is in flight while block i is multiplied; one barrier per
  // block.  LDS reads are issued in batches ahead of the MFMAs that use them (a read costs a few hundred clocks of
  // latency, an MFMA 32): all 16 K fragments of a block before its first score MFMA, the V pieces of the next group
  // of 16 keys before the MFMAs of the present one, those of the first group before the softmax.
  const int li = lane & 15, dgroup = 16 * ((lane >> 4) & 1);  // position in the 16-lane group, the group's first d in a 32-row block
  // LDS addresses, kept few: a K fragment is at [key = 32 t + l32][chunk 2 kk + half] -> this lane's 8 places in
  // its row (the tile t is an immediate offset); a V column piece is at [key][chunk 4 db + c] -> 4 places per lane.
  // (as pointers into both buffers of the pair: the loop adds nothing to them)
  const unsigned char* k_at[2][8];
#pragma unroll
  for (int pb = 0; pb < 2; ++pb)
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) k_at[pb][kk] = buf + pb * BUF_BYTES + l32 * (FA_D * 2) + 16 * k_place(l32, 2 * kk + half);
  const int v_key = 4 * half + (li >> 2);  // the key (within a group of 16) this lane points at for the transposing read
  const unsigned char* v_at[2][4];
#pragma unroll
  for (int pb = 0; pb < 2; ++pb)
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      const int d = 32 * db + dgroup + 4 * (li & 3);
      v_at[pb][db] = buf + pb * BUF_BYTES + K_BYTES + v_key * (FA_D * 2) + 16 * v_place(v_key, d >> 3) + 2 * (d & 4);
    }
  // the 8 pieces (4 blocks of d x two halves of 8 keys) of the group of 16 keys that starts at key `first`
  auto read_v_group = [&](int pb, int first, v4s (&piece)[8]) {
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      // rows first + v_key and 8 further on: (key & 3) is the same, so is the place in the row
      piece[2 * db] = read_v_piece(v_at[pb][db] + first * (FA_D * 2));
      piece[2 * db + 1] = read_v_piece(v_at[pb][db] + (first + 8) * (FA_D * 2));
    }
  };
  issue_block<false>(kres, (uint32_t)first_block * FA_K_BLOCK * FA_D * 2, buf, wave, lane);
  issue_block<true>(vres, (uint32_t)first_block * FA_K_BLOCK * FA_D * 2, buf + K_BYTES, wave, lane);
  // one block of 64 keys; PB = (i - first_block) % 2 (the buffer pair) is a compile-time constant so that the address tables are registers
  auto block = [&](int i, auto pair) {
    constexpr int PB = decltype(pair)::value;
    __syncthreads();  // blocks i of K and V have landed (the barrier drains every wave's loads); buffers of block i - 1 are free
    if (i + 1 < blocks) {
      issue_block<false>(kres, (uint32_t)(i + 1) * FA_K_BLOCK * FA_D * 2, buf + (1 - PB) * BUF_BYTES, wave, lane);
      issue_block<true>(vres, (uint32_t)(i + 1) * FA_K_BLOCK * FA_D * 2, buf + (1 - PB) * BUF_BYTES + K_BYTES, wave, lane);
    }
    const int k0 = i * FA_K_BLOCK;
    if (k0 >= wave_keys || k0 + FA_K_BLOCK <= wave_begin) return;  // no query of this wave sees a key of this block: only the loads and the barrier
    // ---- S^T = K . Q^T : two 32-key tiles -----------------------------------------------------------
    v16f s[2];
    v4s piece[2][8];
    {
      v4i kf[2][8];
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) kf[t][kk] = *reinterpret_cast<const v4i*>(k_at[PB][kk] + t * 32 * (FA_D * 2));
      __builtin_amdgcn_sched_barrier(0);
      __builtin_amdgcn_s_setprio(2);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int r = 0; r < 16; ++r) s[t][r] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 8; ++kk) s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, kf[t][kk]), qf[kk], s[t], 0, 0, 0);
      }
      read_v_group(PB, 0, piece[0]);  // on their way during the softmax
      __builtin_amdgcn_s_setprio(0);
      __builtin_amdgcn_sched_barrier(0);
    }
    // ---- mask, online softmax (in units of log2: exp2(x * scale_log2e - max)) -------------------------------
    const int query = qw + l32;
    const bool all = pipelink_call_mask_all_visible(&view, qw, qw + 31, k0, k0 + FA_K_BLOCK - 1);
    if (!all) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = k0 + 32 * t + 8 * (r / 4) + 4 * half + r % 4;
          if (!pipelink_call_mask_visible(&view, query, key)) s[t][r] = MASKED;
        }
    }
    float block_max = MASKED;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) block_max = fmaxf(block_max, s[t][r]);
    block_max = max_with_other_half(block_max);
    // once a query has seen a key its maximum is a real score, and a masked entry (-1e30) turns into exp2(-huge) = 0
    // by itself
    // The reference point of the exponentials only moves when a score exceeds it by more than 2^RESCALE_SLACK: until
    // then probabilities may be as large as that (harmless in fp32 sums and bf16 operands, and the final division
    // takes it out again), and the accumulated output and sum need no rescaling -- which they otherwise would
    // in most blocks, because some query of the wave sees a new maximum.
    const float top = block_max * p.scale_log2e;
    const float new_max = top > row_max + RESCALE_SLACK ? top : row_max;
    const float alpha = __builtin_amdgcn_exp2f(row_max - new_max);
    row_max = new_max;
    // a query that has not seen a key yet (a window mask: the block's keys are all too old for it) has no real maximum
    // to lean on: its exponentials are taken against +huge instead, which makes every one of them 0
    seen = seen || block_max > 0.5f * MASKED;
    const float reference = seen ? new_max : -MASKED;
    float block_sum = 0.0f;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float e = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][r], p.scale_log2e, -reference));
        s[t][r] = e;
        block_sum += e;
      }
    block_sum = sum_with_other_half(block_sum);
    row_sum = row_sum * alpha + block_sum;
    if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {  // once the maxima have settled nothing needs rescaling
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[db][r] *= alpha;
    }
    // ---- O^T += V^T . P^T : four groups of 16 keys, four 32-row blocks of d ----------------------------
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int gi = 0; gi < 4; ++gi) {
      const int t = gi >> 1, g = gi & 1;
      if (gi + 1 < 4) read_v_group(PB, 16 * (gi + 1), piece[(gi + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
      v8f pf;
#pragma unroll
      for (int e = 0; e < 8; ++e) pf[e] = s[t][8 * g + e];
      const v8bf pb = __builtin_convertvector(pf, v8bf);
#pragma unroll
      for (int db = 0; db < 4; ++db) {
        const v2i lo2 = __builtin_bit_cast(v2i, piece[gi & 1][2 * db]), hi2 = __builtin_bit_cast(v2i, piece[gi & 1][2 * db + 1]);
        const v4i raw = {lo2.x, lo2.y, hi2.x, hi2.y};
        o[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, raw), pb, o[db], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
  };
  for (int i = first_block; i < blocks; i += 2) {
    block(i, std::integral_constant<int, 0>{});
    if (i + 1 < blocks) block(i + 1, std::integral_constant<int, 1>{});
  }
  // ---- O[b][query][h][d] = O^T / row_sum, bf16 ------------------------------------------------------------
  const float inv = row_sum > 0.0f ? __builtin_amdgcn_rcpf(row_sum) : 0.0f;
  uint16_t* orow = p.o + ((int64_t)b * p.seq + qw + l32) * ((int64_t)p.q_heads * FA_D) + (int64_t)h * FA_D;
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int q4 = 0; q4 < 4; ++q4) {
      const v4f f = {o[db][4 * q4] * inv, o[db][4 * q4 + 1] * inv, o[db][4 * q4 + 2] * inv, o[db][4 * q4 + 3] * inv};
      const v4bf packed = __builtin_convertvector(f, v4bf);
      *reinterpret_cast<v2i*>(orow + 32 * db + 8 * q4 + 4 * half) = __builtin_bit_cast(v2i, packed);
    }
}
#else
#include "include/fa_abi.h"
#endif

PL_STAGE("fa.core", "0.1.0");
PL_PARAMS(FaCoreParams);
PL_ROLE(core, fa_core_role_core, 4);
PL_TOPOLOGY(false, "static");
PL_VARIANT(0, {});
PL_CALL(mask_key_count, "mask_key_count",
        "extern \"C\" __device__ int pipelink_call_mask_key_count(const void* view, int q_first, int q_last);");
PL_CALL(mask_key_begin, "mask_key_begin",
        "extern \"C\" __device__ int pipelink_call_mask_key_begin(const void* view, int q_first, int q_last);");
PL_CALL(mask_all_visible, "mask_all_visible",
        "extern \"C\" __device__ int pipelink_call_mask_all_visible(const void* view, int q_first, int q_last, int k_first, int k_last);");
PL_CALL(mask_visible, "mask_visible",
        "extern \"C\" __device__ int pipelink_call_mask_visible(const void* view, int q, int k);");
// two buffers of (K block 16 KB + V block 16 KB)
PL_CLAIM("pipelink_fa_kv", "smem", 2 * 2 * (64 * 128 * 2), 1024, "kernel");
PL_USES("pipelink_fa_kv");
// two workgroups per CU (two waves per SIMD, 256 registers per lane each): one multiplies while the other
// is in its softmax or waits at its barrier; 2 x 67.6 KB of LDS fit
PL_FACT("launch.waves_per_simd", 2);
PL_PRELUDE("include/fa_abi.h");
PL_EMIT_MAIN()
