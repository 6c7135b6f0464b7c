// Recurrent sequence mixers over segments: decayed linear attention, short
// causal convolution with carried taps, and the gated delta rule with a decay
// per key channel. State lives in fp32 slots [slot, H, D, V]; a segment that
// starts a sequence (seg_start == 0) takes its state as zero whatever the
// slot holds, so a reused slot needs no clearing.
//
// Layout of the recurrences: one wave per (segment, head, 64 state columns);
// lane j owns one column of the state (D floats in registers) — the per-token
// update and read-out are then lane-local, and the slot traffic is coalesced
// over j. Splitting the columns over waves keeps a lone long prompt from
// running on H workgroups only.

#include "seq_common.h"

// ---- decayed linear attention ------------------------------------------------
// S <- decay_h S + silu(k) silu(v)^T ; o = S^T silu(q)
template <typename T, int DMAX>
__global__ void __launch_bounds__(WAVE) linear_attn_decay_kernel(
    float* __restrict__ o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const float* __restrict__ decay, float* __restrict__ state, const int* __restrict__ slots,
    const int* __restrict__ cu, const int* __restrict__ seg_start, int H, int D, int V,
    int q_stride, int k_stride, int v_stride) {
  constexpr int PER = (2 * DMAX + WAVE - 1) / WAVE;     // q|k elements staged per lane
  __shared__ float qk[2][2 * DMAX];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, j = blockIdx.z * WAVE + lane;
  const bool live = j < V;
  const int t0 = cu[b], t1 = cu[b + 1];
  float* sp = state + (((int64_t)slots[b] * H + h) * D) * V + j;
  float S[DMAX];
  const bool fresh = seg_start[b] == 0;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (!fresh && live && d < D) ? sp[(int64_t)d * V] : 0.f;
  const float dec = decay[h];
  // software pipeline: token t+1's q, k, v are in flight while token t is computed
  float pre[PER], vpre = 0.f;
  auto fetch = [&](int t) {
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + r * WAVE;
      const bool isq = i < D;
      const int d = isq ? i : i - D;
      pre[r] = i < 2 * D ? ldf((isq ? q + (int64_t)t * q_stride : k + (int64_t)t * k_stride) + (int64_t)h * D + d)
                         : 0.f;
    }
    vpre = live ? ldf(v + (int64_t)t * v_stride + (int64_t)h * V + j) : 0.f;
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float* buf = qk[(t - t0) & 1];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + r * WAVE;
      if (i < 2 * D) buf[i < D ? i : DMAX + (i - D)] = silu_exact(pre[r]);
    }
    const float vj = silu_exact(vpre);
    __syncthreads();    // double-buffered: one barrier per token
    if (t + 1 < t1) fetch(t + 1);
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] = dec * S[d] + buf[DMAX + d] * vj;
        acc += S[d] * buf[d];
      }
    }
    if (live) o[((int64_t)t * H + h) * V + j] = acc;
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d) if (d < D) sp[(int64_t)d * V] = S[d];
  }
}

// ---- short causal convolution + silu ----------------------------------------
// y[t,c] = silu(sum_j w[c,j] * x[t - (K-1-j), c]); inputs before the segment
// come from conv_state [slot, K-1, C] (oldest first), zeros for a fresh sequence.
template <typename T>
__global__ void causal_conv_silu_kernel(T* __restrict__ y, const T* __restrict__ x,
                                        const float* __restrict__ w, const T* __restrict__ conv_state,
                                        const int* __restrict__ slots, const int* __restrict__ cu,
                                        const int* __restrict__ seg_start, const int* __restrict__ token_seg,
                                        int64_t n, int C, int K, int x_stride) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int t = (int)(idx / C), c = (int)(idx - (int64_t)t * C);
    const int b = token_seg[t];
    const int i = t - cu[b];
    const bool fresh = seg_start[b] == 0;
    const T* hist = conv_state + (int64_t)slots[b] * (K - 1) * C;
    float acc = 0.f;
    for (int j = 0; j < K; ++j) {
      const int src = i - (K - 1 - j);
      float xv;
      if (src >= 0) xv = ldf(x + (int64_t)(t - (K - 1 - j)) * x_stride + c);
      else xv = fresh ? 0.f : ldf(hist + (int64_t)(K - 1 + src) * C + c);
      acc += w[(int64_t)c * K + j] * xv;
    }
    stf(y + idx, silu_exact(acc));
  }
}

// new history = last K-1 inputs of (old history ++ this segment's inputs);
// one thread per (segment, channel) reads everything it needs before it writes.
#define CONV_MAX_TAPS 16
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ x, T* __restrict__ conv_state,
                                         const int* __restrict__ slots, const int* __restrict__ cu,
                                         const int* __restrict__ seg_start, int B, int C, int K,
                                         int x_stride) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)B * C) return;
  const int b = (int)(idx / C), c = (int)(idx - (int64_t)b * C);
  const int t0 = cu[b], L = cu[b + 1] - t0;
  if (L == 0) return;
  const bool fresh = seg_start[b] == 0;
  T* hist = conv_state + (int64_t)slots[b] * (K - 1) * C;
  T tmp[CONV_MAX_TAPS];
  for (int j = 0; j < K - 1; ++j) {
    const int src = L - (K - 1) + j;          // index into this segment's inputs
    if (src >= 0) tmp[j] = x[(int64_t)(t0 + src) * x_stride + c];
    else if (fresh) stf(&tmp[j], 0.f);
    else tmp[j] = hist[(int64_t)(K - 1 + src) * C + c];
  }
  for (int j = 0; j < K - 1; ++j) hist[(int64_t)j * C + c] = tmp[j];
}

// ---- gated delta rule, decay per head and key channel ---------------------------
// per token: g_d = exp(-exp(A_h) softplus(a_d + dt_d));  S <- g (.) S (rows)
//            u = beta (v - S^T k^) ; S <- S + k^ u^T ; o = S^T q^
// k^ = k / sqrt(|k|^2 + 1e-6), q^ likewise times D^-1/2; beta = sigmoid(.)
// decay pre-pass, parallel over all (token, head, channel):
//   g = exp(-exp(A_h) softplus(a + dt))
template <typename T>
__global__ void delta_decay_kernel(float* __restrict__ g, const T* __restrict__ a,
                                   const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                   int64_t n, int HD, int D, int a_stride) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t t = i / HD;
    const int c = (int)(i - t * HD);
    const float pre = ldf(a + t * a_stride + c) + dt_bias[c];
    g[i] = expf(-expf(a_log[c / D]) * softplus_exact(pre));
  }
}

template <typename T, int DMAX>
__global__ void __launch_bounds__(WAVE) gated_delta_rule_kernel(
    float* __restrict__ o, const T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
    const T* __restrict__ beta_logit, const float* __restrict__ gdec, float* __restrict__ state,
    const int* __restrict__ slots, const int* __restrict__ cu, const int* __restrict__ seg_start,
    int H, int G, int D, int V, int q_stride, int k_stride, int v_stride, int beta_stride) {
  constexpr int PER = (3 * DMAX + WAVE - 1) / WAVE;     // q|k|g elements staged per lane
  __shared__ float buf_[2][3 * DMAX];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x, j = blockIdx.z * WAVE + lane;
  const int g = h / (H / G);
  const bool live = j < V;
  const int t0 = cu[b], t1 = cu[b + 1];
  float* sp = state + (((int64_t)slots[b] * H + h) * D) * V + j;
  float S[DMAX];
  const bool fresh = seg_start[b] == 0;
#pragma unroll
  for (int d = 0; d < DMAX; ++d) S[d] = (!fresh && live && d < D) ? sp[(int64_t)d * V] : 0.f;
  const float qscale = 1.0f / sqrtf((float)D);
  // software pipeline: token t+1's operands are in flight while token t is computed
  float pre[PER], vpre = 0.f, bpre = 0.f;
  auto fetch = [&](int t) {
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + r * WAVE;
      const int which = i / D, d = i - which * D;
      float val = 0.f;
      if (which == 0) val = ldf(q + (int64_t)t * q_stride + (int64_t)g * D + d);
      else if (which == 1) val = ldf(k + (int64_t)t * k_stride + (int64_t)g * D + d);
      else if (which == 2) val = gdec[((int64_t)t * H + h) * D + d];
      pre[r] = val;
    }
    vpre = live ? ldf(v + (int64_t)t * v_stride + (int64_t)h * V + j) : 0.f;
    bpre = ldf(beta_logit + (int64_t)t * beta_stride + h);
  };
  if (t0 < t1) fetch(t0);
  for (int t = t0; t < t1; ++t) {
    float* buf = buf_[(t - t0) & 1];
#pragma unroll
    for (int r = 0; r < PER; ++r) {
      const int i = lane + r * WAVE;
      const int which = i / D, d = i - which * D;
      if (which < 3) buf[which * DMAX + d] = pre[r];
    }
    const float vj = vpre;
    const float beta = sigmoid_exact(bpre);
    __syncthreads();
    if (t + 1 < t1) fetch(t + 1);
    float pred = 0.f, ksq = 0.f, qsq = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        const float kd = buf[DMAX + d], qd = buf[d];
        S[d] *= buf[2 * DMAX + d];
        pred += S[d] * kd;
        ksq += kd * kd;
        qsq += qd * qd;
      }
    }
    const float rk = 1.0f / sqrtf(ksq + 1e-6f);
    const float rq = qscale / sqrtf(qsq + 1e-6f);
    const float u = beta * (vj - pred * rk) * rk;     // u times the key's normaliser
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < DMAX; ++d) {
      if (d < D) {
        S[d] += buf[DMAX + d] * u;
        acc += S[d] * buf[d];
      }
    }
    if (live) o[((int64_t)t * H + h) * V + j] = acc * rq;
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DMAX; ++d) if (d < D) sp[(int64_t)d * V] = S[d];
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

#define DISPATCH_D(D, ...)                                          \
  if (D <= 32) { constexpr int DMAX = 32; __VA_ARGS__ }             \
  else if (D <= 64) { constexpr int DMAX = 64; __VA_ARGS__ }        \
  else if (D <= 128) { constexpr int DMAX = 128; __VA_ARGS__ }      \
  else { constexpr int DMAX = 256; __VA_ARGS__ }

static inline int col_blocks(int V) { return (V + WAVE - 1) / WAVE; }

extern "C" void seq_launch_linear_attn_decay(float* o, const void* q, const void* k, const void* v,
                                             const float* decay, float* state, const int* slots,
                                             const int* cu, const int* seg_start, int B, int H, int D, int V,
                                             int q_stride, int k_stride, int v_stride, int is_f32,
                                             hipStream_t st) {
  DISPATCH_T(is_f32, DISPATCH_D(D, hipLaunchKernelGGL((linear_attn_decay_kernel<T, DMAX>), dim3(B, H, col_blocks(V)),
                                                      dim3(WAVE), 0, st, o, (const T*)q,
                                                      (const T*)k, (const T*)v, decay, state, slots, cu,
                                                      seg_start, H, D, V, q_stride, k_stride, v_stride);))
}

extern "C" void seq_launch_causal_conv_silu(void* y, const void* x, const float* w, void* conv_state,
                                            const int* slots, const int* cu, const int* seg_start,
                                            const int* token_seg, int T_, int B, int C, int K, int x_stride,
                                            int is_f32, hipStream_t st) {
  const int64_t n = (int64_t)T_ * C;
  const int grid = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  const int grid2 = (int)(((int64_t)B * C + 255) / 256);
  DISPATCH_T(is_f32,
             hipLaunchKernelGGL(causal_conv_silu_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)y, (const T*)x,
                                w, (const T*)conv_state, slots, cu, seg_start, token_seg, n, C, K, x_stride);
             hipLaunchKernelGGL(conv_state_update_kernel<T>, dim3(grid2), dim3(256), 0, st, (const T*)x,
                                (T*)conv_state, slots, cu, seg_start, B, C, K, x_stride);)
}

extern "C" void seq_launch_gated_delta_rule(float* o, const void* q, const void* k, const void* v,
                                            const void* beta_logit, const void* a, const float* dt_bias,
                                            const float* a_log, float* gdec, float* state, const int* slots,
                                            const int* cu, const int* seg_start, int T_, int B, int H, int G,
                                            int D, int V, int q_stride, int k_stride, int v_stride,
                                            int beta_stride, int a_stride, int is_f32, hipStream_t st) {
  const int64_t n = (int64_t)T_ * H * D;
  const int grid = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  DISPATCH_T(is_f32,
             hipLaunchKernelGGL(delta_decay_kernel<T>, dim3(grid), dim3(256), 0, st, gdec, (const T*)a, dt_bias,
                                a_log, n, H * D, D, a_stride);
             DISPATCH_D(D, hipLaunchKernelGGL((gated_delta_rule_kernel<T, DMAX>), dim3(B, H, col_blocks(V)),
                                              dim3(WAVE), 0, st, o, (const T*)q, (const T*)k, (const T*)v,
                                              (const T*)beta_logit, gdec, state, slots, cu, seg_start, H, G, D,
                                              V, q_stride, k_stride, v_stride, beta_stride);))
}
