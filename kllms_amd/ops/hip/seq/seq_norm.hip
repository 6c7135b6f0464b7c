// fp32-residual normalisation kernels and the clamped GLU activation.
// One workgroup per token row; rows are re-read from L1/L2 between passes
// instead of being held in registers, so any width works.

#include "seq_common.h"

// out[t] = rmsnorm(table[ids[t]]) * w   (fp32 residual stream)
template <typename T>
__global__ void embed_rmsnorm_kernel(float* __restrict__ out, const int64_t* __restrict__ ids,
                                     const T* __restrict__ table, const float* __restrict__ w,
                                     int W, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) { float v = ldf(row + i); ss += v * v; }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) out[(int64_t)t * W + i] = ldf(row + i) * r * w[i];
}

// out[t] = rmsnorm(x[t]) * w, x fp32, out in the activation type
template <typename T>
__global__ void rmsnorm_cast_kernel(T* __restrict__ out, const float* __restrict__ x,
                                    const float* __restrict__ w, int W, float eps) {
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * W;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) { float v = x[base + i]; ss += v * v; }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + base + i, x[base + i] * r * w[i]);
}

// Fused sublayer epilogue:
//   y = a                                    (single branch)
//   y = (rms(a) wa + rms(b) wb) / 2          (two branches, DUAL)
//   x += rms(y) * w_post                     (fp32 residual, in place)
//   out = rms(x) * w_next                    (next sublayer's input; optional)
// y is staged in dynamic LDS (W floats).
template <typename T, bool DUAL>
__global__ void sandwich_residual_kernel(float* __restrict__ x, const T* __restrict__ a,
                                         const T* __restrict__ b, const float* __restrict__ wa,
                                         const float* __restrict__ wb, const float* __restrict__ w_post,
                                         const float* __restrict__ w_next, T* __restrict__ out,
                                         int W, float eps) {
  extern __shared__ float ybuf[];
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * W;
  const float invW = 1.0f / (float)W;
  float ssy = 0.f;
  if (DUAL) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float va = ldf(a + base + i), vb = ldf(b + base + i);
      sa += va * va; sb += vb * vb;
    }
    sa = block_sum(sa, scratch);
    sb = block_sum(sb, scratch);
    const float ra = 1.0f / sqrtf(sa * invW + eps), rb = 1.0f / sqrtf(sb * invW + eps);
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float y = 0.5f * (ldf(a + base + i) * ra * wa[i] + ldf(b + base + i) * rb * wb[i]);
      ybuf[i] = y; ssy += y * y;
    }
  } else {
    for (int i = threadIdx.x; i < W; i += blockDim.x) {
      float y = ldf(a + base + i);
      ybuf[i] = y; ssy += y * y;
    }
  }
  ssy = block_sum(ssy, scratch);
  const float ry = 1.0f / sqrtf(ssy * invW + eps);
  float ssx = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {   // each thread re-reads its own ybuf entries
    float v = x[base + i] + ybuf[i] * ry * w_post[i];
    x[base + i] = v; ybuf[i] = v; ssx += v * v;
  }
  if (w_next == nullptr) return;
  ssx = block_sum(ssx, scratch);
  const float rx = 1.0f / sqrtf(ssx * invW + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + base + i, ybuf[i] * rx * w_next[i]);
}

// out[t, g*S + i] = o[t,g,i] / rms(o[t,g,:]) * w[i] * sigmoid(gate[t, g*S + i])
template <typename T>
__global__ void gated_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ o,
                                     const float* __restrict__ w, const T* __restrict__ gate,
                                     int S, int gate_stride, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, g = blockIdx.y, G = gridDim.y;
  const float* row = o + ((int64_t)t * G + g) * S;
  float ss = 0.f;
  for (int i = threadIdx.x; i < S; i += blockDim.x) { float v = row[i]; ss += v * v; }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)S + eps);
  const T* grow = gate + (int64_t)t * gate_stride + (int64_t)g * S;
  T* orow = out + ((int64_t)t * G + g) * S;
  for (int i = threadIdx.x; i < S; i += blockDim.x)
    stf(orow + i, row[i] * r * w[i] * sigmoid_exact(ldf(grow + i)));
}

// y = min(g, lim) * sigmoid(alpha * min(g, lim)) * (clamp(u, -lim, lim) + 1)
template <typename T>
__global__ void clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                   const T* __restrict__ up, int64_t n, int cols, int stride,
                                   float limit, float alpha) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cols, c = i - r * cols;
    float g = fminf(ldf(gate + r * stride + c), limit);
    float u = fminf(fmaxf(ldf(up + r * stride + c), -limit), limit);
    stf(out + i, g * sigmoid_exact(alpha * g) * (u + 1.0f));
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

extern "C" void seq_launch_embed_rmsnorm(float* out, const int64_t* ids, const void* table,
                                         const float* w, int T_, int W, float eps, int is_f32,
                                         hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(embed_rmsnorm_kernel<T>, dim3(T_), dim3(256), 0, st, out, ids,
                                        (const T*)table, w, W, eps);)
}

extern "C" void seq_launch_rmsnorm_cast(void* out, const float* x, const float* w, int T_, int W,
                                        float eps, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(rmsnorm_cast_kernel<T>, dim3(T_), dim3(256), 0, st, (T*)out, x, w,
                                        W, eps);)
}

extern "C" void seq_launch_sandwich_residual(float* x, const void* a, const void* b, const float* wa,
                                             const float* wb, const float* w_post, const float* w_next,
                                             void* out, int T_, int W, float eps, int is_f32,
                                             hipStream_t st) {
  const size_t lds = (size_t)W * sizeof(float);
  if (b != nullptr) {
    DISPATCH_T(is_f32, hipLaunchKernelGGL((sandwich_residual_kernel<T, true>), dim3(T_), dim3(256), lds, st,
                                          x, (const T*)a, (const T*)b, wa, wb, w_post, w_next, (T*)out, W, eps);)
  } else {
    DISPATCH_T(is_f32, hipLaunchKernelGGL((sandwich_residual_kernel<T, false>), dim3(T_), dim3(256), lds, st,
                                          x, (const T*)a, (const T*)b, wa, wb, w_post, w_next, (T*)out, W, eps);)
  }
}

extern "C" void seq_launch_gated_rmsnorm(void* out, const float* o, const float* w, const void* gate,
                                         int T_, int G, int S, int gate_stride, float eps, int is_f32,
                                         hipStream_t st) {
  const int threads = S >= 256 ? 256 : (S > 64 ? 128 : 64);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(gated_rmsnorm_kernel<T>, dim3(T_, G), dim3(threads), 0, st, (T*)out,
                                        o, w, (const T*)gate, S, gate_stride, eps);)
}

extern "C" void seq_launch_clamped_glu(void* out, const void* gate, const void* up, int64_t rows, int cols,
                                       int stride, float limit, float alpha, int is_f32, hipStream_t st) {
  const int64_t n = rows * cols;
  const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(clamped_glu_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)out,
                                        (const T*)gate, (const T*)up, n, cols, stride, limit, alpha);)
}
