// Gated matrix recurrences over segments: wkv (a decay per head, key channel and
// token; the read-out comes before the update and adds a bonus for the current
// token) and mlstm (scalar exponential gates per head and token, stabilised by a
// running maximum, with a normaliser vector carried beside the matrix).
// State lives in fp32 slots; a segment that starts a sequence
// (seg_start == 0) takes its state as zero whatever the slot holds.
//
// Both follow the layout of the other recurrences of this extension: a
// parallel pre-pass turns the projections into the recurrence's fp32 operands
// (decays, gates, the bonus term), then one wave serves (segment, head, 64/NS
// state columns), its NS lane groups splitting the state's rows in registers,
// with a 4-token software pipeline through LDS.

#include "seq_common.h"

__device__ __forceinline__ float logsigmoid_exact(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

// wkv pre-pass, one wave per (token, head):
//   rp = r, kp = k, wp = exp(-exp(d + w0)), vp = v, bonus = sum_d u_d k_d r_d
template <typename T>
__global__ void wkv_prep_kernel(float* __restrict__ rp, float* __restrict__ kp, float* __restrict__ wp,
                                float* __restrict__ vp, float* __restrict__ bonus, const T* __restrict__ r,
                                const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ d,
                                const float* __restrict__ w0, const float* __restrict__ u, int H, int D, int V,
                                int r_stride, int k_stride, int v_stride) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int64_t th = t * H + h;
  float bs = 0.f;
  for (int i = lane; i < D; i += WAVE) {
    const float rv = ldf(r + t * r_stride + (int64_t)h * D + i), kv = ldf(k + t * k_stride + (int64_t)h * D + i);
    rp[th * D + i] = rv;
    kp[th * D + i] = kv;
    wp[th * D + i] = expf(-expf(d[th * D + i] + w0[(int64_t)h * D + i]));
    bs += u[(int64_t)h * D + i] * kv * rv;
  }
  bs = wave_sum(bs);
  if (lane == 0) bonus[th] = bs;
  for (int i = lane; i < V; i += WAVE) vp[th * V + i] = ldf(v + t * v_stride + (int64_t)h * V + i);
}

// mlstm pre-pass, one wave per (token, head):
//   qp = q D^-1/2, kp = k, vp = v, ig = cap tanh((z_i + b_i) / cap),
//   fg = logsigmoid(cap tanh((z_f + b_f) / cap));  z [T, 2H] = input | forget
template <typename T>
__global__ void mlstm_prep_kernel(float* __restrict__ qp, float* __restrict__ kp, float* __restrict__ vp,
                                  float* __restrict__ ig, float* __restrict__ fg, const T* __restrict__ q,
                                  const T* __restrict__ k, const T* __restrict__ v, const float* __restrict__ z,
                                  const float* __restrict__ zb, float cap, int H, int D, int V, int q_stride,
                                  int k_stride, int v_stride) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int64_t th = t * H + h;
  const float qs = 1.0f / sqrtf((float)D);
  for (int i = lane; i < D; i += WAVE) {
    qp[th * D + i] = ldf(q + t * q_stride + (int64_t)h * D + i) * qs;
    kp[th * D + i] = ldf(k + t * k_stride + (int64_t)h * D + i);
  }
  for (int i = lane; i < V; i += WAVE) vp[th * V + i] = ldf(v + t * v_stride + (int64_t)h * V + i);
  if (lane == 0) {
    ig[th] = cap * tanhf((z[t * 2 * H + h] + zb[h]) / cap);
    fg[th] = logsigmoid_exact(cap * tanhf((z[t * 2 * H + H + h] + zb[H + h]) / cap));
  }
}

// MODE 0, wkv:   o = S^T r + bonus v;  S <- diag(w) S + k v^T
//                staged per token: r | k | w;  state [slot, H, D, V]
// MODE 1, mlstm: m' = max(f + m, i); S <- e^(f+m-m') S + e^(i-m') k v~^T; o~ = S^T q
//                with v~ = [v, 1]: the extra column carries the normaliser n,
//                so o~[V] = n . q. staged per token: q | k; state
//                [slot, H, D+1, V+1], row D holds m in every column (each lane
//                reads and writes the copy of its own column). o~ is [T, H, V+1],
//                mt [T, H] receives m'.
template <int DMAX, int NS, int MODE>
__global__ void __launch_bounds__(WAVE) gated_recurrence_kernel(
    float* __restrict__ o, const float* __restrict__ A, const float* __restrict__ Bk,
    const float* __restrict__ Wd, const float* __restrict__ vf, const float* __restrict__ s1,
    const float* __restrict__ s2, float* __restrict__ mt, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu, const int* __restrict__ seg_start, int H, int D,
    int V) {
  constexpr int NV = MODE == 0 ? 3 : 2;
  constexpr int TB = 4;
  constexpr int DR = DMAX / NS, COLS = WAVE / NS;
  constexpr int PER = (NV * DMAX + WAVE - 1) / WAVE;
  __shared__ float buf_[2][TB][NV * DMAX];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int grp = lane / COLS, j = blockIdx.z * COLS + (lane % COLS), d0 = grp * DR;
  const int VC = MODE == 0 ? V : V + 1;             // state columns
  const int RW = MODE == 0 ? D : D + 1;             // state rows
  const bool live = j < VC;
  const bool ones = MODE == 1 && j == V;            // the normaliser's column: v~ = 1
  const int t0 = cu[b], t1 = cu[b + 1];
  if (t1 <= t0) return;
  float* sp = state + (((int64_t)slots[b] * H + h) * RW) * VC + j;
  float S[DR];
  const bool fresh = seg_start[b] == 0;
#pragma unroll
  for (int d = 0; d < DR; ++d) S[d] = (!fresh && live && d0 + d < D) ? sp[(int64_t)(d0 + d) * VC] : 0.f;
  float m = 0.f;
  if (MODE == 1 && !fresh && live) m = sp[(int64_t)D * VC];

  auto step = [&](const float* buf, float vj, float a1, float a2, int t) {
    float acc = 0.f;
    if (MODE == 0) {
#pragma unroll
      for (int d = 0; d < DR; ++d) {
        acc += S[d] * buf[d0 + d];
        S[d] = buf[2 * DMAX + d0 + d] * S[d] + buf[DMAX + d0 + d] * vj;
      }
    } else {
      const float m_new = fmaxf(a2 + m, a1);
      const float fa = expf(a2 + m - m_new), kv = expf(a1 - m_new) * vj;
      m = m_new;
#pragma unroll
      for (int d = 0; d < DR; ++d) {
        S[d] = fa * S[d] + buf[DMAX + d0 + d] * kv;
        acc += S[d] * buf[d0 + d];
      }
    }
#pragma unroll
    for (int off = COLS; off < WAVE; off <<= 1) acc += __shfl_xor(acc, off);
    if (live && grp == 0) o[((int64_t)t * H + h) * VC + j] = MODE == 0 ? acc + a1 * vj : acc;
    if (MODE == 1 && j == 0 && grp == 0) mt[(int64_t)t * H + h] = m;
  };

  if (t1 - t0 == 1) {
    // decode: one row, no pipeline — stage the vectors once (zeros above D)
    float* buf = buf_[0][0];
    for (int i = lane; i < NV * DMAX; i += WAVE) {
      const int which = i / DMAX, d = i - which * DMAX;
      const float* src = which == 0 ? A : which == 1 ? Bk : Wd;
      buf[i] = d < D ? src[((int64_t)t0 * H + h) * D + d] : 0.f;
    }
    const float vj = ones ? 1.f : (live ? vf[((int64_t)t0 * H + h) * V + j] : 0.f);
    const float a1 = s1[(int64_t)t0 * H + h], a2 = MODE == 1 ? s2[(int64_t)t0 * H + h] : 0.f;
    __syncthreads();
    step(buf, vj, a1, a2, t0);
  } else {
    for (int i = lane; i < 2 * TB * NV * DMAX; i += WAVE) (&buf_[0][0][0])[i] = 0.f;   // pad rows stay zero
    __syncthreads();
    float pre[TB][PER], vpre[TB], apre[TB], bpre[TB];
    // where each staged element comes from and goes to, fixed per lane
    const float* src[PER];
    int dst[PER];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + r * WAVE;
      const int which = i / D, d = i - which * D;
      dst[r] = which < NV ? which * DMAX + d : -1;
      src[r] = (which == 0 ? A : which == 1 ? Bk : Wd) + (int64_t)h * D + d;
    }
    const int64_t tstep = (int64_t)H * D;
    auto fetch = [&](int tg) {
#pragma unroll
      for (int u = 0; u < TB; ++u) {
        const int t = tg + u;
        const bool on = t < t1;
#pragma unroll
        for (int r = 0; r < PER; ++r) pre[u][r] = (on && dst[r] >= 0) ? src[r][(int64_t)t * tstep] : 0.f;
        vpre[u] = ones ? 1.f : ((on && live) ? vf[((int64_t)t * H + h) * V + j] : 0.f);
        apre[u] = on ? s1[(int64_t)t * H + h] : 0.f;
        bpre[u] = (MODE == 1 && on) ? s2[(int64_t)t * H + h] : 0.f;
      }
    };
    fetch(t0);
    int flip = 0;
    for (int tg = t0; tg < t1; tg += TB, flip ^= 1) {
      float vj[TB], a1[TB], a2[TB];
#pragma unroll
      for (int u = 0; u < TB; ++u) {
#pragma unroll
        for (int r = 0; r < PER; ++r)
          if (dst[r] >= 0) buf_[flip][u][dst[r]] = pre[u][r];
        vj[u] = vpre[u]; a1[u] = apre[u]; a2[u] = bpre[u];
      }
      __syncthreads();    // double-buffered: one barrier per group
      if (tg + TB < t1) fetch(tg + TB);
#pragma unroll
      for (int u = 0; u < TB; ++u)
        if (tg + u < t1) step(buf_[flip][u], vj[u], a1[u], a2[u], tg + u);
    }
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DR; ++d) if (d0 + d < D) sp[(int64_t)(d0 + d) * VC] = S[d];
    if (MODE == 1 && grp == 0) sp[(int64_t)D * VC] = m;
  }
}

// mlstm read-out: o = o~[:V] / (max(|o~[V]|, e^-m) + 1e-6)
__global__ void mlstm_finish_kernel(float* __restrict__ o, const float* __restrict__ oe,
                                    const float* __restrict__ mt, int64_t n, int V) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / V;
    const int c = (int)(i - th * V);
    const float den = fmaxf(fabsf(oe[th * (V + 1) + V]), expf(-mt[th])) + 1e-6f;
    o[i] = oe[th * (V + 1) + c] / den;
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

#define DISPATCH_D(D, ...)                                          \
  if (D <= 32) { constexpr int DMAX = 32; __VA_ARGS__ }             \
  else if (D <= 64) { constexpr int DMAX = 64; __VA_ARGS__ }        \
  else if (D <= 128) { constexpr int DMAX = 128; __VA_ARGS__ }      \
  else { constexpr int DMAX = 256; __VA_ARGS__ }

#define DISPATCH_NS(ns, ...)                                        \
  if (ns == 2) { constexpr int NS = 2; __VA_ARGS__ }                \
  else if (ns == 4) { constexpr int NS = 4; __VA_ARGS__ }           \
  else { constexpr int NS = 8; __VA_ARGS__ }

// the coarsest split of the state's rows that still gives every SIMD many waves
static inline int pick_split(int B, int H, int V) {
  const int64_t want = 16384;
  for (int ns = 2; ns <= 8; ns *= 2)
    if ((int64_t)B * H * ((V + 64 / ns - 1) / (64 / ns)) >= want) return ns;
  return 8;
}

extern "C" void seq_launch_wkv_recurrence(float* o, const void* r, const void* k, const void* v, const float* d,
                                          const float* w0, const float* u, float* rp, float* kp, float* wp,
                                          float* vp, float* bonus, float* state, const int* slots, const int* cu,
                                          const int* seg_start, int T_, int B, int H, int D, int V, int r_stride,
                                          int k_stride, int v_stride, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(wkv_prep_kernel<T>, dim3(T_, H), dim3(WAVE), 0, st, rp, kp, wp, vp, bonus,
                                        (const T*)r, (const T*)k, (const T*)v, d, w0, u, H, D, V, r_stride,
                                        k_stride, v_stride);)
  const int ns = pick_split(B, H, V);
  DISPATCH_NS(ns, DISPATCH_D(D, hipLaunchKernelGGL((gated_recurrence_kernel<DMAX, NS, 0>),
                                                   dim3(B, H, (V + WAVE / NS - 1) / (WAVE / NS)), dim3(WAVE), 0,
                                                   st, o, rp, kp, wp, vp, bonus, nullptr, nullptr, state, slots,
                                                   cu, seg_start, H, D, V);))
}

extern "C" void seq_launch_mlstm_recurrence(float* o, const void* q, const void* k, const void* v,
                                            const float* z, const float* zb, float cap, float* qp, float* kp,
                                            float* vp, float* ig, float* fg, float* oe, float* mt, float* state,
                                            const int* slots, const int* cu, const int* seg_start, int T_, int B,
                                            int H, int D, int V, int q_stride, int k_stride, int v_stride,
                                            int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(mlstm_prep_kernel<T>, dim3(T_, H), dim3(WAVE), 0, st, qp, kp, vp, ig, fg,
                                        (const T*)q, (const T*)k, (const T*)v, z, zb, cap, H, D, V, q_stride,
                                        k_stride, v_stride);)
  const int ns = pick_split(B, H, V + 1);
  DISPATCH_NS(ns, DISPATCH_D(D, hipLaunchKernelGGL((gated_recurrence_kernel<DMAX, NS, 1>),
                                                   dim3(B, H, (V + 1 + WAVE / NS - 1) / (WAVE / NS)), dim3(WAVE),
                                                   0, st, oe, qp, kp, nullptr, vp, ig, fg, mt, state, slots, cu,
                                                   seg_start, H, D, V);))
  if (o == nullptr) return;          // the caller's norm kernel does the read-out division
  const int64_t n = (int64_t)T_ * H * V;
  const int grid = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  hipLaunchKernelGGL(mlstm_finish_kernel, dim3(grid), dim3(256), 0, st, o, oe, mt, n, V);
}
