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

// dot of a bf16 row of n elements (n % 512 == 0) with the fp32 vector in LDS, by one wave; every lane gets the sum
__device__ __forceinline__ float row_dot(const uint16_t* row, const float* x, int n, int lane) {
  float acc = 0.0f;
  for (int c = lane; c < n / 8; c += 64) {
    const v4i w = *reinterpret_cast<const v4i*>(row + 8 * c);
    const v4f x0 = *reinterpret_cast<const v4f*>(x + 8 * c), x1 = *reinterpret_cast<const v4f*>(x + 8 * c + 4);
    acc += bf16_to_f32((uint32_t)w.x & 0xFFFFu) * x0.x + __uint_as_float((uint32_t)w.x & 0xFFFF0000u) * x0.y;
    acc += bf16_to_f32((uint32_t)w.y & 0xFFFFu) * x0.z + __uint_as_float((uint32_t)w.y & 0xFFFF0000u) * x0.w;
    acc += bf16_to_f32((uint32_t)w.z & 0xFFFFu) * x1.x + __uint_as_float((uint32_t)w.z & 0xFFFF0000u) * x1.y;
    acc += bf16_to_f32((uint32_t)w.w & 0xFFFFu) * x1.z + __uint_as_float((uint32_t)w.w & 0xFFFF0000u) * x1.w;
  }
  return wave_sum(acc);
}
// two rows at once (more loads in flight); sums in a and b
__device__ __forceinline__ void row_dot2(const uint16_t* r0, const uint16_t* r1, const float* x, int n, int lane, float& a, float& b) {
  float acc0 = 0.0f, acc1 = 0.0f;
  for (int c = lane; c < n / 8; c += 64) {
    const v4i w0 = *reinterpret_cast<const v4i*>(r0 + 8 * c), w1 = *reinterpret_cast<const v4i*>(r1 + 8 * c);
    const v4f x0 = *reinterpret_cast<const v4f*>(x + 8 * c), x1 = *reinterpret_cast<const v4f*>(x + 8 * c + 4);
    const float xs[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
    const uint32_t a4[4] = {(uint32_t)w0.x, (uint32_t)w0.y, (uint32_t)w0.z, (uint32_t)w0.w};
    const uint32_t b4[4] = {(uint32_t)w1.x, (uint32_t)w1.y, (uint32_t)w1.z, (uint32_t)w1.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      acc0 += bf16_to_f32(a4[e] & 0xFFFFu) * xs[2 * e] + __uint_as_float(a4[e] & 0xFFFF0000u) * xs[2 * e + 1];
      acc1 += bf16_to_f32(b4[e] & 0xFFFFu) * xs[2 * e] + __uint_as_float(b4[e] & 0xFFFF0000u) * xs[2 * e + 1];
    }
  }
  a = wave_sum(acc0);
  b = wave_sum(acc1);
}
}  // namespace mk
