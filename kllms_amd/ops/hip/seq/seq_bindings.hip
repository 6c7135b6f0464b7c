// PyTorch bindings for the sequence-mixer kernels (kllms_amd._C_seq): shape,
// dtype and stride checks on the host, then a launch on the current stream.
// Activations are bf16 or fp32 (all of one kind per call); the residual
// stream, norm weights, recurrence constants and recurrent state are fp32.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <hip/hip_bf16.h>

extern "C" {
void seq_launch_embed_rmsnorm(float*, const int64_t*, const void*, const float*, int, int, float, int, hipStream_t);
void seq_launch_rmsnorm_cast(void*, const float*, const float*, int, int, float, int, hipStream_t);
void seq_launch_sandwich_residual(float*, const void*, const void*, const float*, const float*, const float*,
                                  const float*, void*, int, int, float, int, hipStream_t);
void seq_launch_gated_rmsnorm(void*, const float*, const float*, const void*, int, int, int, int, float, int,
                              hipStream_t);
void seq_launch_clamped_glu(void*, const void*, const void*, int64_t, int, int, float, float, int, hipStream_t);
void seq_launch_rope_pairs_store(void*, const void*, const void*, const int64_t*, const float*, void*, void*,
                                 const int64_t*, void*, int, int, int, int, int, int, int, int, int, int, int,
                                 hipStream_t);
void seq_launch_attn_blocklocal_paged(void*, const void*, const void*, const void*, const int*, const int*,
                                      const int64_t*, const void*, const int*, int, float, int, int, int, int,
                                      int, int, int, int, int, int, int, hipStream_t);
void seq_launch_head_gate(void*, const void*, int, int, int, int, int, hipStream_t);
void seq_launch_linear_attn_decay(float*, const void*, const void*, const void*, const float*, float*, float*,
                                  const int*, const int*, const int*, int, int, int, int, int, int, int, int,
                                  int, hipStream_t);
void seq_launch_causal_conv_silu(void*, const void*, const float*, void*, const int*, const int*, const int*,
                                 const int*, int, int, int, int, int, int, hipStream_t);
void seq_launch_gated_delta_rule(float*, const void*, const void*, const void*, const void*, const void*,
                                 const float*, const float*, float*, float*, float*, float*, float*, float*,
                                 const int*, const int*, const int*, int, int, int, int, int, int, int, int, int,
                                 int, int, int, hipStream_t);
}

// dense varlen causal MFMA prefill kernel (ops/hip/attn_prefill.hip, also part
// of kllms_amd._C): bf16, head size 128, 8 q-tiles of 32 rows per workgroup
extern "C" __global__ void attn_prefill_kernel(__hip_bfloat16*, const __hip_bfloat16*, const __hip_bfloat16*,
                                               const __hip_bfloat16*, const int*, const int*, const int*, float,
                                               int, int, int, int);

static inline hipStream_t cur_stream() { return at::hip::getCurrentHIPStream().stream(); }

static bool is_act(const torch::Tensor& t) {
  return t.is_cuda() && (t.scalar_type() == at::kBFloat16 || t.scalar_type() == at::kFloat);
}
static int f32flag(const torch::Tensor& t) { return t.scalar_type() == at::kFloat ? 1 : 0; }

#define CHECK_ACT(t) TORCH_CHECK(is_act(t), #t " must be a bf16 or fp32 GPU tensor")
#define CHECK_SAME(t, ref) TORCH_CHECK((t).scalar_type() == (ref).scalar_type(), #t " dtype differs from " #ref)
#define CHECK_F32C(t) \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kFloat && (t).is_contiguous(), #t " must be contiguous fp32 on GPU")
#define CHECK_I32C(t) \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kInt && (t).is_contiguous(), #t " must be contiguous int32 on GPU")
#define CHECK_I64C(t) \
  TORCH_CHECK((t).is_cuda() && (t).scalar_type() == at::kLong && (t).is_contiguous(), #t " must be contiguous int64 on GPU")
// [T, C] or [T, H, D] view whose inner dims are packed; the row stride is free
#define CHECK_ROWS2(t) TORCH_CHECK((t).dim() == 2 && (t).stride(1) == 1, #t " must be a [T, C] row view")
#define CHECK_ROWS3(t) \
  TORCH_CHECK((t).dim() == 3 && (t).stride(2) == 1 && (t).stride(1) == (t).size(2), #t " must be a [T, H, D] row view")

void embed_rmsnorm(torch::Tensor out, torch::Tensor ids, torch::Tensor table, torch::Tensor w, double eps) {
  CHECK_F32C(out); CHECK_I64C(ids); CHECK_ACT(table); CHECK_F32C(w);
  TORCH_CHECK(table.is_contiguous() && table.dim() == 2);
  const int T = ids.numel(), W = table.size(1);
  TORCH_CHECK(out.numel() == (int64_t)T * W && w.numel() == W);
  if (T == 0) return;
  seq_launch_embed_rmsnorm(out.data_ptr<float>(), ids.data_ptr<int64_t>(), table.data_ptr(),
                           w.data_ptr<float>(), T, W, (float)eps, f32flag(table), cur_stream());
}

void rmsnorm_cast(torch::Tensor out, torch::Tensor x, torch::Tensor w, double eps) {
  CHECK_ACT(out); CHECK_F32C(x); CHECK_F32C(w);
  TORCH_CHECK(out.is_contiguous() && out.numel() == x.numel());
  const int W = x.size(-1), T = x.numel() / W;
  TORCH_CHECK(w.numel() == W);
  if (T == 0) return;
  seq_launch_rmsnorm_cast(out.data_ptr(), x.data_ptr<float>(), w.data_ptr<float>(), T, W, (float)eps,
                          f32flag(out), cur_stream());
}

// b / wa / wb: empty tensors for the single-branch form; w_next / out: empty for none
void sandwich_residual(torch::Tensor x, torch::Tensor a, torch::Tensor b, torch::Tensor wa, torch::Tensor wb,
                       torch::Tensor w_post, torch::Tensor w_next, torch::Tensor out, double eps) {
  CHECK_F32C(x); CHECK_ACT(a); CHECK_F32C(w_post);
  TORCH_CHECK(a.is_contiguous() && a.numel() == x.numel());
  const int W = x.size(-1), T = x.numel() / W;
  TORCH_CHECK(w_post.numel() == W);
  TORCH_CHECK((size_t)W * 4 <= 64 * 1024, "width too large for the LDS row buffer");
  const bool dual = b.numel() > 0;
  if (dual) {
    CHECK_SAME(b, a); CHECK_F32C(wa); CHECK_F32C(wb);
    TORCH_CHECK(b.is_cuda() && b.is_contiguous() && b.numel() == a.numel() && wa.numel() == W && wb.numel() == W);
  }
  const bool next = w_next.numel() > 0;
  if (next) {
    CHECK_F32C(w_next); CHECK_SAME(out, a);
    TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.numel() == x.numel() && w_next.numel() == W);
  }
  if (T == 0) return;
  seq_launch_sandwich_residual(x.data_ptr<float>(), a.data_ptr(), dual ? b.data_ptr() : nullptr,
                               dual ? wa.data_ptr<float>() : nullptr, dual ? wb.data_ptr<float>() : nullptr,
                               w_post.data_ptr<float>(), next ? w_next.data_ptr<float>() : nullptr,
                               next ? out.data_ptr() : nullptr, T, W, (float)eps, f32flag(a), cur_stream());
}

void gated_rmsnorm(torch::Tensor out, torch::Tensor o, torch::Tensor w, torch::Tensor gate, double eps) {
  CHECK_ACT(out); CHECK_F32C(o); CHECK_F32C(w); CHECK_ACT(gate); CHECK_SAME(gate, out); CHECK_ROWS2(gate);
  TORCH_CHECK(o.dim() == 3 && out.is_contiguous() && out.numel() == o.numel());
  const int T = o.size(0), G = o.size(1), S = o.size(2);
  TORCH_CHECK(w.numel() == S && gate.size(0) == T && gate.size(1) == (int64_t)G * S);
  if (T == 0) return;
  seq_launch_gated_rmsnorm(out.data_ptr(), o.data_ptr<float>(), w.data_ptr<float>(), gate.data_ptr(), T, G, S,
                           (int)gate.stride(0), (float)eps, f32flag(out), cur_stream());
}

void clamped_glu(torch::Tensor out, torch::Tensor gate, torch::Tensor up, double limit, double alpha) {
  CHECK_ACT(out); CHECK_ACT(gate); CHECK_SAME(up, gate); CHECK_SAME(out, gate); CHECK_ROWS2(gate); CHECK_ROWS2(up);
  TORCH_CHECK(up.is_cuda() && up.sizes() == gate.sizes() && up.stride(0) == gate.stride(0));
  TORCH_CHECK(out.is_contiguous() && out.numel() == gate.numel());
  if (gate.numel() == 0) return;
  seq_launch_clamped_glu(out.data_ptr(), gate.data_ptr(), up.data_ptr(), gate.size(0), (int)gate.size(1),
                         (int)gate.stride(0), (float)limit, (float)alpha, f32flag(gate), cur_stream());
}

// caches: [NB, G, BS, D] / [NB, G, BS, Dv]; v: empty = store the un-rotated key as the value
void rope_pairs_store(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor positions,
                      torch::Tensor inv_freq, torch::Tensor k_cache, torch::Tensor v_cache,
                      torch::Tensor slots, torch::Tensor kv_fresh) {
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_ROWS3(k); CHECK_SAME(k, q); CHECK_SAME(k_cache, q); CHECK_SAME(v_cache, q);
  CHECK_I64C(positions); CHECK_I64C(slots); CHECK_F32C(inv_freq);
  TORCH_CHECK(k.is_cuda() && k_cache.is_cuda() && v_cache.is_cuda() && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  const int T = q.size(0), H = q.size(1), D = q.size(2), G = k.size(1);
  const int BS = k_cache.size(2), Dv = v_cache.size(3), R = inv_freq.numel();
  TORCH_CHECK(k.size(0) == T && k.size(2) == D && k_cache.size(1) == G && k_cache.size(3) == D &&
              v_cache.size(1) == G && v_cache.size(2) == BS && v_cache.size(0) == k_cache.size(0));
  TORCH_CHECK(2 * R <= D, "rotary width exceeds the head size");
  TORCH_CHECK(positions.numel() == T && slots.numel() == T);
  const bool has_v = v.numel() > 0;
  if (has_v) {
    CHECK_ROWS3(v); CHECK_SAME(v, q);
    TORCH_CHECK(v.is_cuda() && v.size(0) == T && v.size(1) == G && v.size(2) == Dv);
  } else {
    TORCH_CHECK(Dv == D, "values-from-keys needs equal key and value sizes");
  }
  const bool fresh = kv_fresh.numel() > 0;
  if (fresh) {
    CHECK_SAME(kv_fresh, q);
    TORCH_CHECK(kv_fresh.is_cuda() && kv_fresh.is_contiguous() && Dv == D &&
                kv_fresh.numel() == (int64_t)T * 2 * G * D, "kv_fresh must be [T, 2, G, D]");
  }
  if (T == 0) return;
  seq_launch_rope_pairs_store(q.data_ptr(), k.data_ptr(), has_v ? v.data_ptr() : nullptr,
                              positions.data_ptr<int64_t>(), inv_freq.data_ptr<float>(), k_cache.data_ptr(),
                              v_cache.data_ptr(), slots.data_ptr<int64_t>(), fresh ? kv_fresh.data_ptr() : nullptr,
                              T, H, G, D, Dv, R, BS,
                              (int)q.stride(0), (int)k.stride(0), has_v ? (int)v.stride(0) : 0, f32flag(q),
                              cur_stream());
}

void attn_blocklocal_paged(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache, torch::Tensor v_cache,
                           torch::Tensor block_tables, torch::Tensor token_seg, torch::Tensor positions,
                           torch::Tensor gate, double scale, int64_t mask_size, torch::Tensor row_map) {
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_SAME(out, q); CHECK_SAME(k_cache, q); CHECK_SAME(v_cache, q);
  CHECK_I32C(block_tables); CHECK_I32C(token_seg); CHECK_I64C(positions);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && k_cache.is_cuda() && v_cache.is_cuda() &&
              k_cache.is_contiguous() && v_cache.is_contiguous() && block_tables.dim() == 2);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k_cache.size(1), BS = k_cache.size(2), Dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == D && H % G == 0 && Dv <= 512 && mask_size >= 0);
  TORCH_CHECK(out.numel() == (int64_t)T * H * Dv && token_seg.numel() == T && positions.numel() == T);
  const bool has_gate = gate.numel() > 0;
  if (has_gate) {
    CHECK_ROWS2(gate); CHECK_SAME(gate, q);
    TORCH_CHECK(gate.is_cuda() && gate.size(0) == T && gate.size(1) == H);
  }
  const bool mapped = row_map.numel() > 0;
  if (mapped) { CHECK_I32C(row_map); TORCH_CHECK(row_map.numel() <= T); }
  if (T == 0) return;
  seq_launch_attn_blocklocal_paged(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                                   block_tables.data_ptr<int>(), token_seg.data_ptr<int>(),
                                   positions.data_ptr<int64_t>(), has_gate ? gate.data_ptr() : nullptr,
                                   mapped ? row_map.data_ptr<int>() : nullptr, (int)row_map.numel(),
                                   (float)scale, (int)mask_size, T, H, G, D, Dv, BS,
                                   (int)block_tables.stride(0), (int)q.stride(0),
                                   has_gate ? (int)gate.stride(0) : 0, f32flag(q), cur_stream());
}

void head_gate(torch::Tensor out, torch::Tensor gate) {
  CHECK_ACT(out); CHECK_ROWS2(gate); CHECK_SAME(gate, out);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 3 && gate.is_cuda() && gate.size(0) == out.size(0) &&
              gate.size(1) == out.size(1));
  if (out.numel() == 0) return;
  seq_launch_head_gate(out.data_ptr(), gate.data_ptr(), (int)out.size(0), (int)out.size(1), (int)out.size(2),
                       (int)gate.stride(0), f32flag(out), cur_stream());
}

// Dense causal attention over packed pieces (each piece attends within
// itself only): q [T,H,128], k/v [T,G,128] row views with one token stride,
// bf16. grp_*: q-tile groups built on the host (8 tiles of 32 rows per
// workgroup, -1 = idle wave). Rows outside every piece are left untouched.
void attn_varlen_mfma(torch::Tensor out, torch::Tensor q, torch::Tensor k, torch::Tensor v,
                      torch::Tensor grp_start, torch::Tensor grp_qpos0, torch::Tensor grp_len, double scale) {
  TORCH_CHECK(q.is_cuda() && q.scalar_type() == at::kBFloat16, "bf16 only");
  CHECK_ROWS3(q); CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_SAME(k, q); CHECK_SAME(v, q); CHECK_SAME(out, q);
  CHECK_I32C(grp_start); CHECK_I32C(grp_qpos0); CHECK_I32C(grp_len);
  const int H = q.size(1), D = q.size(2), G = k.size(1);
  TORCH_CHECK(D == 128 && v.size(2) == 128 && k.size(2) == 128, "head size must be 128");
  TORCH_CHECK(H % G == 0 && v.size(1) == G && k.stride(0) == v.stride(0), "k/v must share heads and token stride");
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.numel() == q.size(0) * (int64_t)H * D);
  const int ngroups = grp_start.numel();
  TORCH_CHECK(grp_qpos0.numel() == (int64_t)ngroups * 8 && grp_len.numel() == ngroups);
  if (ngroups == 0) return;
  hipLaunchKernelGGL(attn_prefill_kernel, dim3(ngroups, H), dim3(512), 0, cur_stream(),
                     (__hip_bfloat16*)out.data_ptr(), (const __hip_bfloat16*)q.data_ptr(),
                     (const __hip_bfloat16*)k.data_ptr(), (const __hip_bfloat16*)v.data_ptr(),
                     grp_start.data_ptr<int>(), grp_len.data_ptr<int>(), grp_qpos0.data_ptr<int>(), (float)scale,
                     H, G, (int)q.stride(0), (int)k.stride(0));
}

static void check_segments(const torch::Tensor& slots, const torch::Tensor& cu, const torch::Tensor& seg_start,
                           const torch::Tensor& state) {
  CHECK_I32C(slots); CHECK_I32C(cu); CHECK_I32C(seg_start);
  TORCH_CHECK(cu.numel() == slots.numel() + 1 && seg_start.numel() == slots.numel());
  TORCH_CHECK(state.is_cuda() && state.is_contiguous());
}

void linear_attn_decay(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor decay,
                       torch::Tensor state, torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start) {
  CHECK_F32C(o); CHECK_ACT(q); CHECK_ROWS3(q); CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_SAME(k, q); CHECK_SAME(v, q);
  CHECK_F32C(decay); CHECK_F32C(state);
  check_segments(slots, cu, seg_start, state);
  const int T = q.size(0), H = q.size(1), D = q.size(2), V = v.size(2), B = slots.numel();
  TORCH_CHECK(k.is_cuda() && v.is_cuda() && k.size(0) == T && v.size(0) == T && k.size(1) == H &&
              v.size(1) == H && k.size(2) == D);
  TORCH_CHECK(D <= 256, "key size above 256 is not supported by the recurrence kernel");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == V);
  TORCH_CHECK(decay.numel() == H && o.numel() == (int64_t)T * H * V);
  if (T == 0 || B == 0) return;
  // silu(q) | silu(k) | silu(v) per (token, head), fp32, from the parallel pre-pass
  auto packed = torch::empty({(int64_t)T, (int64_t)H * (2 * D + V)}, torch::dtype(torch::kFloat).device(q.device()));
  seq_launch_linear_attn_decay(o.data_ptr<float>(), q.data_ptr(), k.data_ptr(), v.data_ptr(),
                               decay.data_ptr<float>(), packed.data_ptr<float>(), state.data_ptr<float>(),
                               slots.data_ptr<int>(), cu.data_ptr<int>(), seg_start.data_ptr<int>(), T, B, H, D,
                               V, (int)q.stride(0), (int)k.stride(0), (int)v.stride(0), f32flag(q),
                               cur_stream());
}

void causal_conv_silu(torch::Tensor y, torch::Tensor x, torch::Tensor w, torch::Tensor conv_state,
                      torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start, torch::Tensor token_seg) {
  CHECK_ACT(x); CHECK_ROWS2(x); CHECK_SAME(y, x); CHECK_SAME(conv_state, x); CHECK_F32C(w); CHECK_I32C(token_seg);
  check_segments(slots, cu, seg_start, conv_state);
  // w: taps-major [K, C], last row = the current token's tap
  TORCH_CHECK(w.dim() == 2);
  const int T = x.size(0), C = x.size(1), K = w.size(0), B = slots.numel();
  TORCH_CHECK(y.is_cuda() && y.is_contiguous() && y.numel() == (int64_t)T * C && w.size(1) == C);
  TORCH_CHECK(K >= 1 && K <= 16, "1..16 convolution taps supported");
  TORCH_CHECK(conv_state.dim() == 3 && conv_state.size(1) == K - 1 && conv_state.size(2) == C);
  TORCH_CHECK(token_seg.numel() == T);
  if (T == 0 || B == 0) return;
  seq_launch_causal_conv_silu(y.data_ptr(), x.data_ptr(), w.data_ptr<float>(), conv_state.data_ptr(),
                              slots.data_ptr<int>(), cu.data_ptr<int>(), seg_start.data_ptr<int>(),
                              token_seg.data_ptr<int>(), T, B, C, K, (int)x.stride(0), f32flag(x), cur_stream());
}

void gated_delta_rule(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor beta,
                      torch::Tensor a, torch::Tensor dt_bias, torch::Tensor a_log, torch::Tensor state,
                      torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start) {
  CHECK_F32C(o); CHECK_ACT(q); CHECK_ROWS3(q); CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_ROWS2(beta); CHECK_ROWS2(a);
  CHECK_SAME(k, q); CHECK_SAME(v, q); CHECK_SAME(beta, q); CHECK_SAME(a, q);
  CHECK_F32C(dt_bias); CHECK_F32C(a_log); CHECK_F32C(state);
  check_segments(slots, cu, seg_start, state);
  const int T = q.size(0), G = q.size(1), D = q.size(2), H = v.size(1), V = v.size(2), B = slots.numel();
  TORCH_CHECK(k.is_cuda() && v.is_cuda() && beta.is_cuda() && a.is_cuda());
  TORCH_CHECK(k.size(0) == T && k.size(1) == G && k.size(2) == D && v.size(0) == T && H % G == 0);
  TORCH_CHECK(beta.size(0) == T && beta.size(1) == H && a.size(0) == T && a.size(1) == (int64_t)H * D);
  TORCH_CHECK(D <= 256, "key size above 256 is not supported by the recurrence kernel");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == V);
  TORCH_CHECK(dt_bias.numel() == (int64_t)H * D && a_log.numel() == H && o.numel() == (int64_t)T * H * V);
  if (T == 0 || B == 0) return;
  // fp32 operands of the recurrence, from the parallel pre-pass: unit q and k,
  // per-channel decays, values, write strengths
  auto f32 = torch::dtype(torch::kFloat).device(q.device());
  auto qn = torch::empty({(int64_t)T, (int64_t)G * D}, f32), kn = torch::empty({(int64_t)T, (int64_t)G * D}, f32);
  auto gd = torch::empty({(int64_t)T, (int64_t)H * D}, f32), vf = torch::empty({(int64_t)T, (int64_t)H * V}, f32);
  auto bt = torch::empty({(int64_t)T, (int64_t)H}, f32);
  seq_launch_gated_delta_rule(o.data_ptr<float>(), q.data_ptr(), k.data_ptr(), v.data_ptr(), beta.data_ptr(),
                              a.data_ptr(), dt_bias.data_ptr<float>(), a_log.data_ptr<float>(),
                              qn.data_ptr<float>(), kn.data_ptr<float>(), gd.data_ptr<float>(),
                              vf.data_ptr<float>(), bt.data_ptr<float>(), state.data_ptr<float>(),
                              slots.data_ptr<int>(),
                              cu.data_ptr<int>(), seg_start.data_ptr<int>(), T, B, H, G, D, V, (int)q.stride(0),
                              (int)k.stride(0), (int)v.stride(0), (int)beta.stride(0), (int)a.stride(0),
                              f32flag(q), cur_stream());
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_rmsnorm", &embed_rmsnorm);
  m.def("rmsnorm_cast", &rmsnorm_cast);
  m.def("sandwich_residual", &sandwich_residual);
  m.def("gated_rmsnorm", &gated_rmsnorm);
  m.def("clamped_glu", &clamped_glu);
  m.def("rope_pairs_store", &rope_pairs_store);
  m.def("attn_blocklocal_paged", &attn_blocklocal_paged);
  m.def("head_gate", &head_gate);
  m.def("attn_varlen_mfma", &attn_varlen_mfma);
  m.def("linear_attn_decay", &linear_attn_decay);
  m.def("causal_conv_silu", &causal_conv_silu);
  m.def("gated_delta_rule", &gated_delta_rule);
}
