// Shared helpers for the sequence-mixer kernels (kllms_amd._C_seq): the
// listed-layer hybrid family keeps its residual stream, norms, attention
// weights and recurrent state in fp32; activations that feed GEMMs are bf16
// (serving) or fp32 (exact mode), so every kernel is templated on that type.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

typedef unsigned short bfraw;  // bf16 bit pattern

__device__ __forceinline__ float ldf(const float* p) { return *p; }
__device__ __forceinline__ float ldf(const bfraw* p) {
  union { float f; uint32_t i; } c;
  c.i = ((uint32_t)*p) << 16;
  return c.f;
}
__device__ __forceinline__ void stf(float* p, float v) { *p = v; }
__device__ __forceinline__ void stf(bfraw* p, float v) {
  // round-to-nearest-even, as torch's float -> bfloat16 cast
  union { float f; uint32_t i; } c;
  c.f = v;
  uint32_t x = c.i;
  if ((x & 0x7fffffffu) > 0x7f800000u) { *p = (bfraw)((x >> 16) | 0x40); return; }
  x += 0x7fffu + ((x >> 16) & 1u);
  *p = (bfraw)(x >> 16);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}

// sum over the whole block (<= 16 waves); every thread gets the total
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wid = threadIdx.x / WAVE;
  v = wave_sum(v);
  if (lane == 0) scratch[wid] = v;
  __syncthreads();
  const int nw = (blockDim.x + WAVE - 1) / WAVE;
  v = lane < nw ? scratch[lane] : 0.0f;
  v = wave_sum(v);
  __syncthreads();
  return v;
}

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + __expf(-x)); }
__device__ __forceinline__ float sigmoid_exact(float x) { return 1.0f / (1.0f + expf(-x)); }
__device__ __forceinline__ float silu_exact(float x) { return x / (1.0f + expf(-x)); }
__device__ __forceinline__ float softplus_exact(float x) { return x > 20.0f ? x : log1pf(expf(x)); }
