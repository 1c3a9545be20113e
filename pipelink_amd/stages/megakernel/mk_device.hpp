// Device helpers shared by the megakernel's op packages.
#pragma once
#include <hip/hip_runtime.h>
#include "include/mk_abi.h"

extern "C" __device__ int pipelink_mk_vec();  // byte offset of the workgroup's activation vector in dynamic LDS
extern __shared__ __attribute__((aligned(1024))) unsigned char pipelink_smem[];

namespace mk {
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ const MkModel& model(const void* view) {
  return *static_cast<const MkModel*>(static_cast<const pipelink_host_view*>(view)->residue);
}
__device__ __forceinline__ float* vec() { return reinterpret_cast<float*>(pipelink_smem + pipelink_mk_vec()); }
// Activations that one workgroup writes and others read after a grid barrier (x, qkv, the attention partials, h)
// are accessed at device scope, word by word: such a store goes through to memory and such a load does not trust a
// line another XCD may have changed, so the barrier itself needs no cache write-back or invalidation.
__device__ __forceinline__ float shared_load(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// four consecutive floats of such a buffer (16-byte aligned): one buffer load at device scope (cache policy bit 4)
__device__ __forceinline__ v4f shared_load4(const float* base, int index, int count) {
  const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base), 0, count * 4, 0x00020000);
  return __builtin_bit_cast(v4f, __builtin_amdgcn_raw_buffer_load_b128(r, index * 4, 0, 16));
}
__device__ __forceinline__ void shared_store(float* p, float v) { __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); }
__device__ __forceinline__ float bf16_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// where a layer's weights start, and the pieces inside a layer (bf16 elements)
struct Layer {
  const uint16_t *attn_norm, *wqkv, *wo, *ffn_norm, *wgate, *wup, *wdown;
};
__device__ __forceinline__ Layer layer_of(const MkModel& m, int layer) {
  const int64_t d = m.d, qkv = (int64_t)(m.hq + 2 * m.hkv) * MK_HEAD_DIM, od = (int64_t)m.hq * MK_HEAD_DIM;
  const uint16_t* p = m.weights + (int64_t)layer * mk_layer_elems(&m);
  Layer l;
  l.attn_norm = p; p += d;
  l.wqkv = p; p += qkv * d;
  l.wo = p; p += d * od;
  l.ffn_norm = p; p += d;
  l.wgate = p; p += (int64_t)m.dff * d;
  l.wup = p; p += (int64_t)m.dff * d;
  l.wdown = p;
  return l;
}
__device__ __forceinline__ const uint16_t* final_norm(const MkModel& m) { return m.weights + (int64_t)m.layers * mk_layer_elems(&m); }
__device__ __forceinline__ const uint16_t* lm_head(const MkModel& m) { return final_norm(m) + m.d; }

// this workgroup's contiguous share [first, last) of `total` rows
__device__ __forceinline__ void my_rows(int total, int& first, int& last) {
  const int per = (total + (int)gridDim.x - 1) / (int)gridDim.x;
  first = min((int)blockIdx.x * per, total);
  last = min(first + per, total);
}

// Lane exchanges inside a row of 16 lanes as DPP operands of the add itself (no LDS round trip as a shuffle is):
// 0xB1 / 0x4E swap neighbours / pairs inside a quad, 0x141 mirrors each half row (swaps its quads), 0x140 mirrors
// the row (swaps its halves), 0x104 / 0x108 read the lane four / eight further on, 0x128 the lane eight away (rotating).
template <int CTRL>
__device__ __forceinline__ float dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}
// sum over the wave, in every lane
__device__ __forceinline__ float wave_sum(float v) {
  v += dpp<0xB1>(v);
  v += dpp<0x4E>(v);
  v += dpp<0x141>(v);
  v += dpp<0x140>(v);  // every lane: the sum of its row
  return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, dpp<0xB1>(v));
  v = fmaxf(v, dpp<0x4E>(v));
  v = fmaxf(v, dpp<0x141>(v));
  v = fmaxf(v, dpp<0x140>(v));
  return fmaxf(fmaxf(lane_value(v, 0), lane_value(v, 16)), fmaxf(lane_value(v, 32), lane_value(v, 48)));
}
// sum over each aligned group of eight lanes, valid in the group's first lane
__device__ __forceinline__ float sum8_first(float v) {
  v += dpp<0xB1>(v);
  v += dpp<0x4E>(v);
  v += dpp<0x104>(v);
  return v;
}

__device__ __forceinline__ float dot8(const v4i w, const v4f x0, const v4f x1) {
  const uint32_t u[4] = {(uint32_t)w.x, (uint32_t)w.y, (uint32_t)w.z, (uint32_t)w.w};
  const float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
  float acc = 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) acc += bf16_to_f32(u[e] & 0xFFFFu) * xs[2 * e] + __uint_as_float(u[e] & 0xFFFF0000u) * xs[2 * e + 1];
  return acc;
}

// One pass over R consecutive bf16 rows (`pitch` elements apart, n elements each, n % 8 == 0): lane `c0` takes the
// 8-element chunks c0, c0 + 64, c0 + 128, c0 + 192 of every row.  rows_load issues the R x 4 sixteen-byte loads,
// rows_fma uses them against the fp32 vector in LDS: between the two a caller can do what does not need them.
template <int R>
__device__ __forceinline__ void rows_load(const uint16_t* rows, int64_t pitch, int n, int c0, v4i (&w)[R][4]) {
#pragma unroll
  for (int r = 0; r < R; ++r)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const v4i zero = {0, 0, 0, 0};
      // weights pass through once per token: loaded as non-temporal, they do not push the activations out of the L2
      w[r][j] = c0 + 64 * j < n / 8 ? __builtin_nontemporal_load(reinterpret_cast<const v4i*>(rows + r * pitch + 8 * (c0 + 64 * j))) : zero;
    }
}
template <int R>
__device__ __forceinline__ void rows_fma(const v4i (&w)[R][4], const float* x, int n, int c0, float (&acc)[R]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (c0 + 64 * j >= n / 8) break;  // rows shorter than 2048 elements
    const v4f x0 = *reinterpret_cast<const v4f*>(x + 8 * (c0 + 64 * j)), x1 = *reinterpret_cast<const v4f*>(x + 8 * (c0 + 64 * j) + 4);
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] += dot8(w[r][j], x0, x1);
  }
}
template <int R>
__device__ __forceinline__ void wave_sums(float (&acc)[R]) {
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = wave_sum(acc[r]);
}

// Dots of R consecutive bf16 rows with the fp32 vector in LDS, by one wave; every lane gets the sums.  `first` holds
// the loads of the first pass (c0 = lane) if the caller issued them already.
template <int R>
__device__ __forceinline__ void rows_dot(const uint16_t* rows, int64_t pitch, const float* x, int n, int lane, float (&sum)[R],
                                         const v4i (*first)[R][4] = nullptr) {
#pragma unroll
  for (int r = 0; r < R; ++r) sum[r] = 0.0f;
  int c0 = lane;
  if (first) {
    rows_fma<R>(*first, x, n, c0, sum);
    c0 += 256;
  }
  for (; c0 < n / 8; c0 += 256) {
    v4i w[R][4];
    rows_load<R>(rows, pitch, n, c0, w);
    rows_fma<R>(w, x, n, c0, sum);
  }
  wave_sums<R>(sum);
}

// y(row) for this workgroup's rows [first, last) of a matrix with rows of n elements: waves take groups of R rows.
// Rows of up to 2048 elements are one pass each, and then a wave loads its next group before it sums the present one.
// `ready` is called once, by every thread, after the wave's first loads have been issued and before x is read:
// the place to wait for x.
template <int R, typename Emit, typename Ready>
__device__ __forceinline__ void matvec(const uint16_t* w, int n, const float* x, int first, int last, Emit&& emit, Ready&& ready) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int r = first + R * wave;
  auto finish = [&](const v4i (&loaded)[R][4], int row) {
    float sum[R];
    rows_dot<R>(w + (int64_t)row * n, n, x, n, lane, sum, &loaded);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < R; ++i) emit(row + i, sum[i]);
    }
  };
  if (r + R <= last) {
    v4i wa[R][4], wb[R][4];
    rows_load<R>(w + (int64_t)r * n, n, n, lane, wa);
    ready();
    for (;;) {
      int next = r + 4 * R;
      bool more = next + R <= last;
      if (more) rows_load<R>(w + (int64_t)next * n, n, n, lane, wb);
      finish(wa, r);
      r = next;
      if (!more) break;
      next = r + 4 * R;
      more = next + R <= last;
      if (more) rows_load<R>(w + (int64_t)next * n, n, n, lane, wa);
      finish(wb, r);
      r = next;
      if (!more) break;
    }
  } else {
    ready();
  }
  for (; r < last; ++r) {  // a last group with fewer than R rows
    float sum[1];
    rows_dot<1>(w + (int64_t)r * n, n, x, n, lane, sum);
    if (lane == 0) emit(r, sum[0]);
  }
}
// y(row) for R consecutive rows (R <= 8) by the whole workgroup: the four waves take a quarter of the columns each
// (n % 32 == 0), so that R x 4 loads per lane are in flight on every wave; the partial sums meet in `scratch`
// (4 x R floats of LDS).  split_load issues a wave's first pass; matvec_split (all threads call it) does the rest
// and ends with threads < count emitting one row each.
template <int R>
__device__ __forceinline__ void split_load(const uint16_t* rows, int n, v4i (&w)[R][4]) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  rows_load<R>(rows + wave * (n / 4), n, n / 4, lane, w);
}
template <int R, typename Emit>
__device__ __forceinline__ void matvec(const uint16_t* w, int n, const float* x, int first, int last, Emit&& emit) {
  matvec<R>(w, n, x, first, last, emit, [] {});
}
template <int R, typename Emit>
__device__ __forceinline__ void matvec_split(const uint16_t* rows, int n, const float* x, float* scratch, int count, const v4i (&loaded)[R][4], Emit&& emit) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, q = n / 4;
  float sum[R];
  rows_dot<R>(rows + wave * q, n, x + wave * q, q, lane, sum, &loaded);
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < R; ++i) scratch[wave * R + i] = sum[i];
  }
  __syncthreads();
  if ((int)threadIdx.x < count) emit((int)threadIdx.x, scratch[threadIdx.x] + scratch[R + threadIdx.x] + scratch[2 * R + threadIdx.x] + scratch[3 * R + threadIdx.x]);
  __syncthreads();
}
}  // namespace mk
