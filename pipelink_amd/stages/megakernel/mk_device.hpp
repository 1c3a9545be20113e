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

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1) v += __shfl_xor(v, s);
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

// Dots of R consecutive bf16 rows (n elements each, n % 512 == 0, `pitch` elements apart) with the fp32 vector in
// LDS, by one wave: all R x 4 loads of a pass are issued before any is used, so a lane keeps up to 4 R sixteen-byte
// loads in flight.  Every lane gets the sums.
template <int R>
__device__ __forceinline__ void rows_dot(const uint16_t* rows, int64_t pitch, const float* x, int n, int lane, float (&sum)[R]) {
  float acc[R];
#pragma unroll
  for (int r = 0; r < R; ++r) acc[r] = 0.0f;
  for (int c0 = lane; c0 < n / 8; c0 += 256) {  // four chunks of 8 elements per lane and pass
    v4i w[R][4];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const v4i zero = {0, 0, 0, 0};
        w[r][j] = c0 + 64 * j < n / 8 ? *reinterpret_cast<const v4i*>(rows + r * pitch + 8 * (c0 + 64 * j)) : zero;
      }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (c0 + 64 * j >= n / 8) break;  // rows shorter than 2048 elements
      const v4f x0 = *reinterpret_cast<const v4f*>(x + 8 * (c0 + 64 * j)), x1 = *reinterpret_cast<const v4f*>(x + 8 * (c0 + 64 * j) + 4);
#pragma unroll
      for (int r = 0; r < R; ++r) acc[r] += dot8(w[r][j], x0, x1);
    }
  }
#pragma unroll
  for (int s = 32; s >= 1; s >>= 1)
#pragma unroll
    for (int r = 0; r < R; ++r) acc[r] += __shfl_xor(acc[r], s);
#pragma unroll
  for (int r = 0; r < R; ++r) sum[r] = acc[r];
}

// y(row) for this workgroup's rows [first, last) of a matrix with rows of n elements: waves take groups of R rows
template <int R, typename Emit>
__device__ __forceinline__ void matvec(const uint16_t* w, int n, const float* x, int first, int last, Emit&& emit) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int r = first + R * wave;
  for (; r + R <= last; r += 4 * R) {
    float sum[R];
    rows_dot<R>(w + (int64_t)r * n, n, x, n, lane, sum);
    if (lane == 0) {
#pragma unroll
      for (int i = 0; i < R; ++i) emit(r + i, sum[i]);
    }
  }
  for (; r < last; ++r) {  // a last group with fewer than R rows
    float sum[1];
    rows_dot<1>(w + (int64_t)r * n, n, x, n, lane, sum);
    if (lane == 0) emit(r, sum[0]);
  }
}
// y(row) for R consecutive rows (R <= 8): the four waves take a quarter of the columns each (n % 2048 == 0 or the
// quarter is a multiple of 512), so that R x 4 loads per lane are in flight on every wave; partial sums meet in
// `scratch` (4 x R floats of LDS).  All threads must call it; ends with a barrier-protected emit by threads < R.
template <int R, typename Emit>
__device__ __forceinline__ void matvec_split(const uint16_t* rows, int n, const float* x, float* scratch, int count, Emit&& emit) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, q = n / 4;
  float sum[R];
  rows_dot<R>(rows + wave * q, n, x + wave * q, q, lane, sum);
  if (lane == 0) {
#pragma unroll
    for (int i = 0; i < R; ++i) scratch[wave * R + i] = sum[i];
  }
  __syncthreads();
  if ((int)threadIdx.x < count) emit((int)threadIdx.x, scratch[threadIdx.x] + scratch[R + threadIdx.x] + scratch[2 * R + threadIdx.x] + scratch[3 * R + threadIdx.x]);
  __syncthreads();
}
}  // namespace mk
