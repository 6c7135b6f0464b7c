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

// 8-element vector access (16 B of bf16, 2 x 16 B of fp32). Callers check on
// the host that the pointers are 16-byte aligned and that row lengths and
// strides are multiples of 8 before taking a kernel that uses these.
__device__ __forceinline__ void ld8(const float* p, float v[8]) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
__device__ __forceinline__ void ld8(const bfraw* p, float v[8]) {
  const uint4 a = *reinterpret_cast<const uint4*>(p);
  const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    union { float f; uint32_t u; } lo, hi;
    lo.u = w[i] << 16; hi.u = w[i] & 0xffff0000u;
    v[2 * i] = lo.f; v[2 * i + 1] = hi.f;
  }
}
__device__ __forceinline__ void st8(float* p, const float v[8]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}
__device__ __forceinline__ uint32_t bf_bits(float f) {
  union { float f; uint32_t i; } c;
  c.f = f;
  uint32_t x = c.i;
  if ((x & 0x7fffffffu) > 0x7f800000u) return (x >> 16) | 0x40;
  x += 0x7fffu + ((x >> 16) & 1u);
  return x >> 16;
}
__device__ __forceinline__ void st8(bfraw* p, const float v[8]) {
  uint4 a;
  a.x = bf_bits(v[0]) | (bf_bits(v[1]) << 16);
  a.y = bf_bits(v[2]) | (bf_bits(v[3]) << 16);
  a.z = bf_bits(v[4]) | (bf_bits(v[5]) << 16);
  a.w = bf_bits(v[6]) | (bf_bits(v[7]) << 16);
  *reinterpret_cast<uint4*>(p) = a;
}
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }
