// Measurement aid for the roofline: what the matrix pipe alone sustains on this board.  Built into a library of its
// own (libplk_bench_probe.so) that only the benchmark loads; the drop-in library does not export it.
//
// The published FP8 peak (5.0 PFLOP/s) is 256 CUs x 4 SIMDs x 2048 flop per clock at 2.4 GHz.
// A kernel that keeps the MFMA pipe busy with non-trivial operands draws the board's full
// power budget and is clocked down, so the rate a GEMM can approach is lower and depends on the
// operand bits.  plk_probe_mfma_fp8 runs nothing but back-to-back
// v_mfma_scale_f32_32x32x64_f8f6f4 -- the instruction the grouped GEMM is made of -- on every
// SIMD, 16 independent accumulators per wave, operands held in registers: no LDS, no memory
// traffic.  Timed by the caller, it gives that ceiling for random e4m3 operands and, with
// zero operands, the rate at the unthrottled clock.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));

__device__ uint32_t mix(uint32_t x) {  // integer hash: operand bits that do not repeat across lanes
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// e4m3 has two NaN codes (0x7f, 0xff); clearing bit 0 of such a byte leaves a finite number
__device__ uint32_t finite_e4m3x4(uint32_t w) {
  uint32_t nan = w & (w >> 1) & (w >> 2) & (w >> 3) & (w >> 4) & (w >> 5) & (w >> 6) & 0x01010101u;
  return w & ~nan;
}

__global__ void __launch_bounds__(256) mfma_burn(int iters, int zero_operands, uint32_t seed, float* sink) {
  v8i a[4], b[4];
  for (int i = 0; i < 4; ++i)
    for (int k = 0; k < 8; ++k) {
      const uint32_t id = ((blockIdx.x * 256u + threadIdx.x) * 8u + i) * 16u + k;
      a[i][k] = zero_operands ? 0 : (int)finite_e4m3x4(mix(id ^ seed));
      b[i][k] = zero_operands ? 0 : (int)finite_e4m3x4(mix(id * 2654435761u + seed));
    }
  v16f acc[16];
  for (int i = 0; i < 16; ++i)
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.0f;
  const int scale = 0x7f7f7f7f;  // e8m0 127 = 1.0 in every byte
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int i = 0; i < 16; ++i)
      acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i / 4], b[i % 4], acc[i], 0, 0, 0, scale, 0, scale);
  }
  float s = 0.0f;
  for (int i = 0; i < 16; ++i)
    for (int r = 0; r < 16; ++r) s += acc[i][r];
  if (s == 12345.678f) sink[0] = s;  // keeps the chain alive without a store on the usual path
}
}  // namespace

// Launches `workgroups` workgroups of 256 threads (one wave per SIMD) that each issue iters * 16 MFMAs per wave on
// operands held in registers -- random finite e4m3 bytes, or zeros -- and nothing else:
// flop = workgroups * 4 * iters * 16 * 131072.  `sink` is 4 bytes of device memory (never written in practice).
// Returns 0, -1 for arguments out of range, or the hipError_t of the launch.
extern "C" int plk_probe_mfma_fp8(int32_t workgroups, int32_t iters, int32_t zero_operands, uint64_t sink, void* stream) {
  if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 22) || !sink) return -1;
  // 100 KB of dynamic LDS keeps it to one workgroup per CU: one wave per SIMD, like the GEMM
  hipLaunchKernelGGL(mfma_burn, dim3((unsigned)workgroups), dim3(256), 100 * 1024, static_cast<hipStream_t>(stream),
                     (int)iters, (int)zero_operands, 0x9e3779b9u, reinterpret_cast<float*>(sink));
  return (int)hipGetLastError();
}
