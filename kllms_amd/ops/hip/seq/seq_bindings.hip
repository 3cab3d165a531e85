// PyTorch bindings for the sequence-mixer kernels (kllms_amd._C_seq): shape,
// dtype and stride checks on the host, then a launch on the current stream.
// Activations are bf16 or fp32 (all of one kind per call); the residual
// stream, norm weights, recurrence constants and recurrent state are fp32.

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>
#include <hip/hip_bf16.h>

extern "C" {
void seq_launch_embed_rmsnorm(float*, const int64_t*, const void*, const float*, const void*, const int64_t*, int,
                              int, float, int, hipStream_t);
void seq_launch_gelu_tanh(void*, const void*, int64_t, int, int, int, hipStream_t);
void seq_launch_scale_softcap(float*, int64_t, float, float, hipStream_t);
void seq_launch_scale_rows(void*, const void*, const int*, const float*, int, int, int, hipStream_t);
void seq_launch_moe_spread_rows(void*, const void*, const int*, const float*, int, int, int, int, int, hipStream_t);
void seq_launch_latent_kv_store(void*, const void*, const float*, float, const int64_t*, const float*, void*,
                                const int64_t*, int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_attn_latent_paged(void*, const void*, const void*, const void*, const int*, const int*,
                                  const int64_t*, const void*, float, int, int, int, int, int, int, int, int,
                                  int64_t, int64_t, int, int, int, int, float*, float*, int, int, hipStream_t);
void seq_launch_rmsnorm_cast(void*, const float*, const float*, int, int, float, int, hipStream_t);
void seq_launch_sandwich_residual(float*, const void*, const void*, const float*, const float*, const float*,
                                  const float*, void*, int, int, float, int, hipStream_t);
void seq_launch_gated_rmsnorm(void*, const float*, const float*, const void*, int, int, int, int, float, int,
                              int, hipStream_t);
void seq_launch_gated_act(void*, const void*, const void*, int64_t, int, int, float, float, float, int,
                          hipStream_t);
void seq_launch_rope_pairs_store(void*, const void*, const void*, const int64_t*, const float*, void*, void*,
                                 const int64_t*, void*, int, int, int, int, int, int, int, int, int, int, int,
                                 hipStream_t);
void seq_launch_attn_masked_paged(void*, const void*, const void*, const void*, const int*, const int*,
                                  const int64_t*, const void*, const int*, int, const float*, const float*, int,
                                  int, float, int, float*, float*, float, int, int, int, int, int,
                                  int, int, int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_qk_fullnorm_rope_store(void*, const void*, const void*, const float*, const float*, float,
                                       const int64_t*, const float*, void*, void*, const int64_t*, int, int, int,
                                       int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_pool_kv_update(const void*, const void*, float*, float*, const int*, const int*, const int64_t*,
                               const int*, int, int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_ln_residual_mix(float*, const float*, const void*, const float*, float*, float*, const float*, int,
                                int64_t, int, int, float, int, hipStream_t);
void seq_launch_ln_canon(void*, const float*, const float*, const float*, const float*, float*, int64_t,
                         const int*, const int*, const int*, const int*, int, int, int, int, int, hipStream_t);
void seq_launch_ssd_recurrence(float*, const void*, const void*, const void*, const void*, const float*,
                               const float*, const float*, float*, float*, float*, const int*, const int*,
                               const int*, int, int, int, int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_qk_norm_store(void*, const void*, const void*, const float*, const float*, float, void*, void*,
                              const int64_t*, int, int, int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_embed_bigram(float*, const int64_t*, const void*, const void*, float, int, int, int, int*,
                             const int*, const int*, const int*, const int*, int, int, int, int, hipStream_t);
void seq_launch_group_norm_pair(float*, const void*, const void*, const float*, const float*, void*, void*, int,
                                int, int, float, int, hipStream_t);
void seq_launch_cast_concat(void*, float*, const float*, const void*, const void*, int, int, int, hipStream_t);
void seq_launch_head_rmsnorm_gate(void*, const float*, const float*, const void*, const float*, int, int, int,
                                  int, float, int, int, hipStream_t);
void seq_launch_token_shift_mix(void*, float*, const void*, const float*, void*, const int*, const int*,
                                const int*, const int*, int, int, int, int, int, int, hipStream_t);
void seq_launch_moe_route(int*, float*, int*, const float*, const void*, const float*, const float*, int, int, int,
                          int, int, int, int, int, int, int, hipStream_t);
void seq_launch_moe_combine(void*, const void*, const void*, const int*, const float*, const void*, const void*,
                            int, int, int, int, int, hipStream_t);
void seq_launch_wkv_recurrence(float*, const void*, const void*, const void*, const float*, const float*,
                               const float*, float*, float*, float*, float*, float*, float*, const int*,
                               const int*, const int*, int, int, int, int, int, int, int, int, int, hipStream_t);
void seq_launch_mlstm_recurrence(float*, const void*, const void*, const void*, const float*, const float*, float,
                                 float*, float*, float*, float*, float*, float*, float*, float*, const int*,
                                 const int*, const int*, int, int, int, int, int, int, int, int, int,
                                 hipStream_t);
void seq_launch_head_gate(void*, const void*, int, int, int, int, int, hipStream_t);
void seq_launch_linear_attn_decay(float*, const void*, const void*, const void*, const float*, float*, float*,
                                  const int*, const int*, const int*, int, int, int, int, int, int, int, int,
                                  int, hipStream_t);
void seq_launch_causal_conv_silu(void*, const void*, const float*, void*, const int*, const int*, const int*,
                                 const int*, const float*, int, int, int, int, int, int, hipStream_t);
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

// pos_table / positions: empty tensors for an embedding without position rows
void embed_rmsnorm(torch::Tensor out, torch::Tensor ids, torch::Tensor table, torch::Tensor w, double eps,
                   torch::Tensor pos_table, torch::Tensor positions) {
  CHECK_F32C(out); CHECK_I64C(ids); CHECK_ACT(table); CHECK_F32C(w);
  TORCH_CHECK(table.is_contiguous() && table.dim() == 2);
  const int T = ids.numel(), W = table.size(1);
  TORCH_CHECK(out.numel() == (int64_t)T * W && w.numel() == W);
  const bool pos = pos_table.numel() > 0;
  if (pos) {
    CHECK_ACT(pos_table); CHECK_SAME(pos_table, table); CHECK_I64C(positions);
    TORCH_CHECK(pos_table.is_contiguous() && pos_table.dim() == 2 && pos_table.size(1) == W && positions.numel() == T);
  }
  if (T == 0) return;
  seq_launch_embed_rmsnorm(out.data_ptr<float>(), ids.data_ptr<int64_t>(), table.data_ptr(),
                           w.data_ptr<float>(), pos ? pos_table.data_ptr() : nullptr,
                           pos ? positions.data_ptr<int64_t>() : nullptr, T, W, (float)eps, f32flag(table),
                           cur_stream());
}

void gelu_tanh(torch::Tensor out, torch::Tensor x) {
  CHECK_ACT(out); CHECK_ACT(x); CHECK_SAME(x, out); CHECK_ROWS2(x);
  TORCH_CHECK(out.is_contiguous() && out.numel() == x.numel());
  if (x.numel() == 0) return;
  seq_launch_gelu_tanh(out.data_ptr(), x.data_ptr(), x.size(0), (int)x.size(1), (int)x.stride(0), f32flag(out),
                       cur_stream());
}

void scale_softcap(torch::Tensor z, double scale, double cap) {
  CHECK_F32C(z);
  if (z.numel() == 0) return;
  seq_launch_scale_softcap(z.data_ptr<float>(), z.numel(), (float)scale, (float)cap, cur_stream());
}

void scale_rows(torch::Tensor out, torch::Tensor h, torch::Tensor src_row, torch::Tensor scale) {
  CHECK_ACT(out); CHECK_ACT(h); CHECK_SAME(h, out); CHECK_I32C(src_row); CHECK_F32C(scale);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && out.dim() == 2 && out.is_contiguous());
  const int n = src_row.numel(), W = h.size(1);
  TORCH_CHECK(out.size(0) == n && out.size(1) == W && scale.numel() == n);
  if (n == 0) return;
  seq_launch_scale_rows(out.data_ptr(), h.data_ptr(), src_row.data_ptr<int>(), scale.data_ptr<float>(), n, W,
                        f32flag(out), cur_stream());
}

// out [E, T, W]: expert e's input rows, w[t, j] * h[t] where e is row t's j-th choice, else zero
void moe_spread_rows(torch::Tensor out, torch::Tensor h, torch::Tensor idx, torch::Tensor w) {
  CHECK_ACT(out); CHECK_ACT(h); CHECK_SAME(h, out); CHECK_I32C(idx); CHECK_F32C(w);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && out.dim() == 3 && out.is_contiguous());
  const int E = out.size(0), T = h.size(0), W = h.size(1);
  TORCH_CHECK(out.size(1) == T && out.size(2) == W && idx.dim() == 2 && idx.size(0) == T && w.numel() == idx.numel());
  TORCH_CHECK((int64_t)E * T < (1LL << 31));
  if (E * T == 0) return;
  seq_launch_moe_spread_rows(out.data_ptr(), h.data_ptr(), idx.data_ptr<int>(), w.data_ptr<float>(), E, T, W,
                             (int)idx.size(1), f32flag(out), cur_stream());
}

// q [T, H, D + R] row view (rotated in place), dkv [T, C + R] row view,
// cache [NB, 1, BS, C + R] contiguous
void latent_kv_store(torch::Tensor q, torch::Tensor dkv, torch::Tensor w, double eps, torch::Tensor positions,
                     torch::Tensor inv_freq, torch::Tensor cache, torch::Tensor slots, int64_t nope_dim) {
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_ACT(dkv); CHECK_SAME(dkv, q); CHECK_ROWS2(dkv); CHECK_F32C(w);
  CHECK_I64C(positions); CHECK_F32C(inv_freq); CHECK_ACT(cache); CHECK_SAME(cache, q); CHECK_I64C(slots);
  const int T = q.size(0), H = q.size(1), D = (int)nope_dim, R = (int)q.size(2) - D;
  const int C = (int)dkv.size(1) - R;
  TORCH_CHECK(D >= 0 && R >= 0 && R % 2 == 0 && C >= 1 && inv_freq.numel() == R / 2 && w.numel() == C);
  TORCH_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(1) == 1 && cache.size(3) == C + R);
  TORCH_CHECK(dkv.size(0) == T && positions.numel() == T && slots.numel() == T);
  if (T == 0) return;
  seq_launch_latent_kv_store(q.data_ptr(), dkv.data_ptr(), w.data_ptr<float>(), (float)eps,
                             positions.data_ptr<int64_t>(), inv_freq.data_ptr<float>(), cache.data_ptr(),
                             slots.data_ptr<int64_t>(), T, H, D, R, C, (int)q.stride(0), (int)dkv.stride(0),
                             f32flag(q), cur_stream());
}

// out [T, H, C] contiguous; q_abs [T, H, C] with free row and head strides;
// q [T, H, D + R] row view; gate [T, H] row view or empty; tile_rows: rows per
// workgroup of the matrix-unit kernel (0 = as many as fit), use_mfma false =
// the plain kernel
void attn_latent_paged(torch::Tensor out, torch::Tensor q_abs, torch::Tensor q, torch::Tensor cache,
                       torch::Tensor block_tables, torch::Tensor token_seg, torch::Tensor positions,
                       torch::Tensor gate, double scale, int64_t mask_size, int64_t nope_dim, int64_t tile_rows,
                       bool use_mfma, torch::Tensor part_o, torch::Tensor part_ml) {
  CHECK_ACT(out); CHECK_ACT(q_abs); CHECK_SAME(q_abs, out); CHECK_ACT(q); CHECK_SAME(q, out); CHECK_ROWS3(q);
  CHECK_ACT(cache); CHECK_SAME(cache, out); CHECK_I32C(token_seg); CHECK_I64C(positions);
  TORCH_CHECK(block_tables.is_cuda() && block_tables.scalar_type() == at::kInt && block_tables.dim() == 2 &&
              block_tables.stride(1) == 1);
  const int T = q.size(0), H = q.size(1), D = (int)nope_dim, R = (int)q.size(2) - D;
  TORCH_CHECK(q_abs.dim() == 3 && q_abs.size(0) == T && q_abs.size(1) == H && q_abs.stride(2) == 1);
  const int C = q_abs.size(2);
  TORCH_CHECK(D >= 0 && R >= 0 && C >= 1 && C <= 1024, "latent size out of range for the attention kernel");
  TORCH_CHECK(cache.dim() == 4 && cache.is_contiguous() && cache.size(1) == 1 && cache.size(3) == C + R);
  TORCH_CHECK(out.is_contiguous() && out.dim() == 3 && out.size(0) == T && out.size(1) == H && out.size(2) == C);
  TORCH_CHECK(token_seg.numel() == T && positions.numel() == T && mask_size >= 0);
  TORCH_CHECK((size_t)(C + R + 128) * 4 <= 64 * 1024);
  const bool g = gate.numel() > 0;
  if (g) { CHECK_ACT(gate); CHECK_SAME(gate, out); CHECK_ROWS2(gate); TORCH_CHECK(gate.size(0) == T && gate.size(1) == H); }
  // key shares: part_o [T, H, nsplit, C], part_ml [T, H, nsplit, 2] fp32, or empty
  int nsplit = 1;
  if (part_o.numel() > 0) {
    CHECK_F32C(part_o); CHECK_F32C(part_ml);
    TORCH_CHECK(part_o.dim() == 4 && part_o.size(0) == T && part_o.size(1) == H && part_o.size(3) == C);
    nsplit = (int)part_o.size(2);
    TORCH_CHECK(nsplit >= 1 && nsplit <= 64 && part_ml.numel() == (int64_t)T * H * nsplit * 2);
  }
  if (T == 0) return;
  seq_launch_attn_latent_paged(out.data_ptr(), q_abs.data_ptr(), q.data_ptr(), cache.data_ptr(),
                               block_tables.data_ptr<int>(), token_seg.data_ptr<int>(),
                               positions.data_ptr<int64_t>(), g ? gate.data_ptr() : nullptr, (float)scale,
                               (int)mask_size, T, H, D, R, C, (int)cache.size(2), (int)block_tables.stride(0),
                               q_abs.stride(0), q_abs.stride(1), (int)q.stride(0), g ? (int)gate.stride(0) : 0,
                               (int)tile_rows, use_mfma ? 1 : 0, nsplit > 1 ? part_o.data_ptr<float>() : nullptr,
                               nsplit > 1 ? part_ml.data_ptr<float>() : nullptr, nsplit, f32flag(out),
                               cur_stream());
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
  const bool want = out.numel() > 0;            // without w_next: the stream itself, cast
  TORCH_CHECK(want || !next, "w_next needs an output tensor");
  if (next) { CHECK_F32C(w_next); TORCH_CHECK(w_next.numel() == W); }
  if (want) {
    CHECK_SAME(out, a);
    TORCH_CHECK(out.is_cuda() && out.is_contiguous() && out.numel() == x.numel());
  }
  if (T == 0) return;
  seq_launch_sandwich_residual(x.data_ptr<float>(), a.data_ptr(), dual ? b.data_ptr() : nullptr,
                               dual ? wa.data_ptr<float>() : nullptr, dual ? wb.data_ptr<float>() : nullptr,
                               w_post.data_ptr<float>(), next ? w_next.data_ptr<float>() : nullptr,
                               want ? out.data_ptr() : nullptr, T, W, (float)eps, f32flag(a), cur_stream());
}

// gate_first: out = rms(o * silu(gate)) * w with w [G * S]; else out = rms(o) * w * sigmoid(gate) with w [S]
void gated_rmsnorm(torch::Tensor out, torch::Tensor o, torch::Tensor w, torch::Tensor gate, double eps,
                   bool gate_first) {
  CHECK_ACT(out); CHECK_F32C(o); CHECK_F32C(w); CHECK_ACT(gate); CHECK_SAME(gate, out); CHECK_ROWS2(gate);
  TORCH_CHECK(o.dim() == 3 && out.is_contiguous() && out.numel() == o.numel());
  const int T = o.size(0), G = o.size(1), S = o.size(2);
  TORCH_CHECK(w.numel() == (gate_first ? (int64_t)G * S : S) && gate.size(0) == T &&
              gate.size(1) == (int64_t)G * S);
  if (T == 0) return;
  seq_launch_gated_rmsnorm(out.data_ptr(), o.data_ptr<float>(), w.data_ptr<float>(), gate.data_ptr(), T, G, S,
                           (int)gate.stride(0), (float)eps, gate_first ? 1 : 0, f32flag(out), cur_stream());
}

void gated_act(torch::Tensor out, torch::Tensor gate, torch::Tensor up, double limit, double alpha,
               double up_bias) {
  CHECK_ACT(out); CHECK_ACT(gate); CHECK_SAME(up, gate); CHECK_SAME(out, gate); CHECK_ROWS2(gate); CHECK_ROWS2(up);
  TORCH_CHECK(up.is_cuda() && up.sizes() == gate.sizes() && up.stride(0) == gate.stride(0));
  TORCH_CHECK(out.is_contiguous() && out.numel() == gate.numel());
  if (gate.numel() == 0) return;
  seq_launch_gated_act(out.data_ptr(), gate.data_ptr(), up.data_ptr(), gate.size(0), (int)gate.size(1),
                       (int)gate.stride(0), (float)limit, (float)alpha, (float)up_bias, f32flag(gate),
                       cur_stream());
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

// gate: empty, [T, H] (one logit per head) or [T, H*Dv] (one per output element)
void attn_masked_paged(torch::Tensor out, torch::Tensor q, torch::Tensor k_cache, torch::Tensor v_cache,
                       torch::Tensor block_tables, torch::Tensor token_seg, torch::Tensor positions,
                       torch::Tensor gate, double scale, int64_t mask_kind, int64_t mask_size,
                       int64_t keep_first, bool sink, torch::Tensor row_map, torch::Tensor pool_k,
                       torch::Tensor pool_v, int64_t run, double softcap, torch::Tensor part_o,
                       torch::Tensor part_ml) {
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_SAME(out, q); CHECK_SAME(k_cache, q); CHECK_SAME(v_cache, q);
  CHECK_I32C(block_tables); CHECK_I32C(token_seg); CHECK_I64C(positions);
  TORCH_CHECK(out.is_cuda() && out.is_contiguous() && k_cache.is_cuda() && v_cache.is_cuda() &&
              k_cache.is_contiguous() && v_cache.is_contiguous() && block_tables.dim() == 2);
  const int T = q.size(0), H = q.size(1), D = q.size(2);
  const int G = k_cache.size(1), BS = k_cache.size(2), Dv = v_cache.size(3);
  TORCH_CHECK(k_cache.size(3) == D && H % G == 0 && Dv <= 512 && mask_size >= 0 && keep_first >= 0);
  TORCH_CHECK(mask_kind >= 0 && mask_kind <= 2,
              "mask_kind: 0 = aligned blocks, 1 = sliding window, 2 = sliding window + pooled runs");
  // pooled caches [NB, G, ceil(BS / run), D|Dv] fp32, used by mask_kind 2 with run > 0
  const bool pooled = mask_kind == 2 && run > 0 && mask_size > 0;
  int PB = 0;
  if (pooled) {
    CHECK_F32C(pool_k); CHECK_F32C(pool_v);
    PB = (BS + (int)run - 1) / (int)run;
    TORCH_CHECK(pool_k.dim() == 4 && pool_v.dim() == 4 && pool_k.size(0) == k_cache.size(0) &&
                pool_v.size(0) == k_cache.size(0) && pool_k.size(1) == G && pool_v.size(1) == G &&
                pool_k.size(2) == PB && pool_v.size(2) == PB && pool_k.size(3) == D && pool_v.size(3) == Dv);
  }
  TORCH_CHECK(softcap >= 0.0);
  // key shares: part_o [T, H, Z, Dv], part_ml [T, H, Z, 2] fp32 scratch; empty = one workgroup per (row, head)
  int nsplit = 1;
  if (part_o.numel() > 0) {
    CHECK_F32C(part_o); CHECK_F32C(part_ml);
    TORCH_CHECK(part_o.dim() == 4 && part_o.size(0) == T && part_o.size(1) == H && part_o.size(3) == Dv &&
                part_ml.numel() == (int64_t)T * H * part_o.size(2) * 2 && part_o.size(2) <= 64);
    nsplit = part_o.size(2);
  }
  TORCH_CHECK(out.numel() == (int64_t)T * H * Dv && token_seg.numel() == T && positions.numel() == T);
  int gate_kind = 0;
  if (gate.numel() > 0) {
    CHECK_ROWS2(gate); CHECK_SAME(gate, q);
    TORCH_CHECK(gate.is_cuda() && gate.size(0) == T && (gate.size(1) == H || gate.size(1) == (int64_t)H * Dv));
    gate_kind = (gate.size(1) == (int64_t)H * Dv && Dv > 1) ? 2 : 1;
  }
  const bool mapped = row_map.numel() > 0;
  if (mapped) { CHECK_I32C(row_map); TORCH_CHECK(row_map.numel() <= T); }
  if (T == 0) return;
  seq_launch_attn_masked_paged(out.data_ptr(), q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
                               block_tables.data_ptr<int>(), token_seg.data_ptr<int>(),
                               positions.data_ptr<int64_t>(), gate_kind ? gate.data_ptr() : nullptr,
                               mapped ? row_map.data_ptr<int>() : nullptr, (int)row_map.numel(),
                               pooled ? pool_k.data_ptr<float>() : nullptr,
                               pooled ? pool_v.data_ptr<float>() : nullptr, pooled ? (int)run : 0, PB,
                               (float)softcap, nsplit, nsplit > 1 ? part_o.data_ptr<float>() : nullptr,
                               nsplit > 1 ? part_ml.data_ptr<float>() : nullptr, (float)scale, (int)mask_kind, (int)mask_size, (int)keep_first, sink ? 1 : 0,
                               gate_kind, T, H, G, D, Dv, BS,
                               (int)block_tables.stride(0), (int)q.stride(0),
                               gate_kind ? (int)gate.stride(0) : 0, f32flag(q), cur_stream());
}

void qk_norm_store(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor wq, torch::Tensor wk,
                   double eps, torch::Tensor k_cache, torch::Tensor v_cache, torch::Tensor slots) {
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_SAME(k, q); CHECK_SAME(v, q);
  CHECK_SAME(k_cache, q); CHECK_SAME(v_cache, q); CHECK_F32C(wq); CHECK_F32C(wk); CHECK_I64C(slots);
  TORCH_CHECK(k.is_cuda() && v.is_cuda() && k_cache.is_cuda() && v_cache.is_cuda() && k_cache.is_contiguous() &&
              v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
  const int T = q.size(0), H = q.size(1), D = q.size(2), G = k.size(1);
  const int BS = k_cache.size(2), Dv = v_cache.size(3);
  TORCH_CHECK(k.size(0) == T && k.size(2) == D && v.size(0) == T && v.size(1) == G && v.size(2) == Dv);
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D && v_cache.size(1) == G && v_cache.size(2) == BS &&
              v_cache.size(0) == k_cache.size(0));
  TORCH_CHECK(wq.numel() == D && wk.numel() == D && slots.numel() == T);
  if (T == 0) return;
  seq_launch_qk_norm_store(q.data_ptr(), k.data_ptr(), v.data_ptr(), wq.data_ptr<float>(), wk.data_ptr<float>(),
                           (float)eps, k_cache.data_ptr(), v_cache.data_ptr(), slots.data_ptr<int64_t>(), T, H,
                           G, D, Dv, BS, (int)q.stride(0), (int)k.stride(0), (int)v.stride(0), f32flag(q),
                           cur_stream());
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
                      torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start, torch::Tensor token_seg,
                      torch::Tensor bias) {
  CHECK_ACT(x); CHECK_ROWS2(x); CHECK_SAME(y, x); CHECK_SAME(conv_state, x); CHECK_F32C(w); CHECK_I32C(token_seg);
  const bool has_bias = bias.numel() > 0;
  if (has_bias) { CHECK_F32C(bias); TORCH_CHECK(bias.numel() == x.size(1)); }
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
                              token_seg.data_ptr<int>(), has_bias ? bias.data_ptr<float>() : nullptr, T, B, C, K,
                              (int)x.stride(0), f32flag(x), cur_stream());
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

// ---- parallel-layer family ------------------------------------------------------

static void check_segments(const torch::Tensor& slots, const torch::Tensor& cu, const torch::Tensor& seg_start,
                           int T) {
  CHECK_I32C(slots); CHECK_I32C(cu); CHECK_I32C(seg_start);
  TORCH_CHECK(cu.numel() == slots.numel() + 1 && seg_start.numel() == slots.numel());
}

void embed_bigram(torch::Tensor out, torch::Tensor ids, torch::Tensor table, torch::Tensor bigram, double scale,
                  int64_t mul_prev, int64_t mul_cur, int64_t buckets, torch::Tensor tok_state,
                  torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start, torch::Tensor token_seg) {
  CHECK_F32C(out); CHECK_I64C(ids); CHECK_ACT(table);
  TORCH_CHECK(table.is_contiguous() && table.dim() == 2);
  const int T = ids.numel(), W = table.size(1), B = slots.numel();
  TORCH_CHECK(out.numel() == (int64_t)T * W);
  check_segments(slots, cu, seg_start, T);
  CHECK_I32C(token_seg);
  TORCH_CHECK(token_seg.numel() == T);
  const bool has = bigram.numel() > 0;
  if (has) {
    CHECK_ACT(bigram); CHECK_SAME(bigram, table); CHECK_I32C(tok_state);
    TORCH_CHECK(bigram.is_contiguous() && bigram.dim() == 2 && bigram.size(1) == W && buckets >= 1 &&
                bigram.size(0) == buckets + 1);
  }
  if (T == 0) return;
  seq_launch_embed_bigram(out.data_ptr<float>(), ids.data_ptr<int64_t>(), table.data_ptr(),
                          has ? bigram.data_ptr() : nullptr, (float)scale, (int)mul_prev, (int)mul_cur,
                          (int)buckets, has ? tok_state.data_ptr<int>() : nullptr, slots.data_ptr<int>(),
                          cu.data_ptr<int>(), seg_start.data_ptr<int>(), token_seg.data_ptr<int>(), T, B, W,
                          f32flag(table), cur_stream());
}

void group_norm_pair(torch::Tensor x, torch::Tensor a, torch::Tensor b, torch::Tensor w1, torch::Tensor w2,
                     torch::Tensor out1, torch::Tensor out2, int64_t groups, double eps) {
  CHECK_F32C(x); CHECK_F32C(w1); CHECK_ACT(out1);
  TORCH_CHECK(x.dim() == 2 && out1.is_contiguous() && out1.numel() == x.numel());
  const int T = x.size(0), W = x.size(1);
  TORCH_CHECK(groups >= 1 && W % groups == 0 && w1.numel() == W && W <= 15360 && groups <= 1024);
  const bool has_a = a.numel() > 0, has_b = b.numel() > 0, two = out2.numel() > 0;
  TORCH_CHECK(has_a || !has_b, "second branch without a first");
  if (has_a) { CHECK_ACT(a); CHECK_SAME(a, out1); TORCH_CHECK(a.is_contiguous() && a.numel() == x.numel()); }
  if (has_b) { CHECK_ACT(b); CHECK_SAME(b, out1); TORCH_CHECK(b.is_contiguous() && b.numel() == x.numel()); }
  if (two) {
    CHECK_ACT(out2); CHECK_SAME(out2, out1); CHECK_F32C(w2);
    TORCH_CHECK(out2.is_contiguous() && out2.numel() == x.numel() && w2.numel() == W);
  }
  if (T == 0) return;
  seq_launch_group_norm_pair(x.data_ptr<float>(), has_a ? a.data_ptr() : nullptr, has_b ? b.data_ptr() : nullptr,
                             w1.data_ptr<float>(), two ? w2.data_ptr<float>() : nullptr, out1.data_ptr(),
                             two ? out2.data_ptr() : nullptr, T, W, (int)groups, (float)eps, f32flag(out1),
                             cur_stream());
}

void cast_concat(torch::Tensor out, torch::Tensor x, torch::Tensor x0, torch::Tensor a, torch::Tensor b) {
  CHECK_ACT(out); CHECK_F32C(x); CHECK_F32C(x0);
  TORCH_CHECK(x.dim() == 2 && x0.sizes() == x.sizes() && out.is_contiguous() && out.numel() == 2 * x.numel());
  const int T = x.size(0), W = x.size(1);
  const bool has_a = a.numel() > 0, has_b = b.numel() > 0;
  TORCH_CHECK(has_a || !has_b, "second branch without a first");
  if (has_a) { CHECK_ACT(a); CHECK_SAME(a, out); TORCH_CHECK(a.is_contiguous() && a.numel() == x.numel()); }
  if (has_b) { CHECK_ACT(b); CHECK_SAME(b, out); TORCH_CHECK(b.is_contiguous() && b.numel() == x.numel()); }
  if (T == 0) return;
  seq_launch_cast_concat(out.data_ptr(), x.data_ptr<float>(), x0.data_ptr<float>(),
                         has_a ? a.data_ptr() : nullptr, has_b ? b.data_ptr() : nullptr, T, W, f32flag(out),
                         cur_stream());
}

// mt: empty, or [T, H] running maxima — then o is [T, H, S + 1] with the normaliser as its last column
void head_rmsnorm_gate(torch::Tensor out, torch::Tensor o, torch::Tensor w, torch::Tensor gate, double eps,
                       int64_t gate_act, torch::Tensor mt) {
  CHECK_ACT(out); CHECK_F32C(o); CHECK_F32C(w); CHECK_ACT(gate); CHECK_SAME(gate, out); CHECK_ROWS2(gate);
  const bool ext = mt.numel() > 0;
  TORCH_CHECK(o.dim() == 3 && out.is_contiguous());
  const int T = o.size(0), H = o.size(1), S = (int)o.size(2) - (ext ? 1 : 0);
  TORCH_CHECK(S >= 1 && out.numel() == (int64_t)T * H * S);
  TORCH_CHECK(w.numel() == (int64_t)H * S && gate.size(0) == T && gate.size(1) == (int64_t)H * S);
  TORCH_CHECK(gate_act == 0 || gate_act == 1, "gate_act: 0 = sigmoid, 1 = silu");
  if (ext) { CHECK_F32C(mt); TORCH_CHECK(mt.numel() == (int64_t)T * H); }
  if (T == 0) return;
  seq_launch_head_rmsnorm_gate(out.data_ptr(), o.data_ptr<float>(), w.data_ptr<float>(), gate.data_ptr(),
                               ext ? mt.data_ptr<float>() : nullptr, T, H, S, (int)gate.stride(0), (float)eps,
                               (int)gate_act, f32flag(out), cur_stream());
}

void token_shift_mix(torch::Tensor act, torch::Tensor f32, torch::Tensor h, torch::Tensor mu,
                     torch::Tensor shift_state, torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start,
                     torch::Tensor token_seg) {
  CHECK_ACT(h); CHECK_F32C(mu); CHECK_SAME(shift_state, h); CHECK_I32C(token_seg);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && mu.dim() == 2 && shift_state.is_cuda() &&
              shift_state.is_contiguous() && shift_state.dim() == 2);
  const int T = h.size(0), W = h.size(1), n = mu.size(0), B = slots.numel();
  check_segments(slots, cu, seg_start, T);
  TORCH_CHECK(mu.size(1) == W && shift_state.size(1) == W && token_seg.numel() == T);
  const int n_act = act.numel() > 0 ? (int)act.size(0) : 0;
  if (n_act > 0) { CHECK_ACT(act); CHECK_SAME(act, h); TORCH_CHECK(act.is_contiguous()); }
  if (n - n_act > 0) { CHECK_F32C(f32); }
  TORCH_CHECK(act.numel() == (int64_t)n_act * T * W && f32.numel() == (int64_t)(n - n_act) * T * W);
  if (T == 0) return;
  seq_launch_token_shift_mix(n_act ? act.data_ptr() : nullptr, n - n_act ? f32.data_ptr<float>() : nullptr,
                             h.data_ptr(), mu.data_ptr<float>(), shift_state.data_ptr(), slots.data_ptr<int>(),
                             cu.data_ptr<int>(), seg_start.data_ptr<int>(), token_seg.data_ptr<int>(), T, B, W,
                             n, n_act, f32flag(h), cur_stream());
}

// x: fp32 logits [T, N] (router empty), or the rows h [T, W] with router [N, W] fp32 — then the logits are
// computed in the kernel. rowidx: empty, or [T, top] for the all-experts form over `experts` real experts.
void moe_route(torch::Tensor idx, torch::Tensor w, torch::Tensor rowidx, torch::Tensor x, torch::Tensor router,
               torch::Tensor corr, int64_t top, int64_t gc, int64_t gk, int64_t experts, int64_t score_kind,
               bool renorm) {
  CHECK_I32C(idx); CHECK_F32C(w);
  TORCH_CHECK(x.dim() == 2 && x.is_cuda() && x.is_contiguous());
  const bool fused = router.numel() > 0;
  const bool has_corr = corr.numel() > 0;          // empty: the choice is made on the plain scores
  if (has_corr) CHECK_F32C(corr);
  const int T = x.size(0), N = fused ? router.size(0) : x.size(1);
  TORCH_CHECK(!has_corr || corr.numel() == N);
  TORCH_CHECK(score_kind == 0 || score_kind == 1);
  int W = 0;
  if (fused) {
    CHECK_ACT(x); CHECK_F32C(router);
    W = x.size(1);
    TORCH_CHECK(router.dim() == 2 && router.size(0) == N && router.size(1) == W);
  } else {
    CHECK_F32C(x);
    TORCH_CHECK(x.size(1) == N);
  }
  TORCH_CHECK(N >= 1 && N <= 256, "the router kernel serves up to 256 outputs");
  TORCH_CHECK(gc >= 1 && N % gc == 0 && gk >= 1 && gk <= gc && top >= 1 && top <= (N / gc) * gk && top <= 64);
  TORCH_CHECK(idx.numel() == (int64_t)T * top && w.numel() == (int64_t)T * top);
  const bool rows = rowidx.numel() > 0;
  if (rows) { CHECK_I32C(rowidx); TORCH_CHECK(rowidx.numel() == (int64_t)T * top && experts * T < (1LL << 31)); }
  if (T == 0) return;
  seq_launch_moe_route(idx.data_ptr<int>(), w.data_ptr<float>(), rows ? rowidx.data_ptr<int>() : nullptr,
                       fused ? nullptr : x.data_ptr<float>(), fused ? x.data_ptr() : nullptr,
                       fused ? router.data_ptr<float>() : nullptr, has_corr ? corr.data_ptr<float>() : nullptr, T,
                       N, W, (int)top, (int)gc, (int)gk, (int)experts, (int)score_kind, renorm ? 1 : 0,
                       fused ? f32flag(x) : 1, cur_stream());
}

// w: empty = unweighted; extra [T, W] / extra_gate ([T] view, any stride): empty = none
void moe_combine(torch::Tensor out, torch::Tensor rows, torch::Tensor h, torch::Tensor rowidx, torch::Tensor w,
                 torch::Tensor extra, torch::Tensor extra_gate) {
  CHECK_ACT(out); CHECK_ACT(rows); CHECK_ACT(h); CHECK_SAME(rows, out); CHECK_SAME(h, out);
  CHECK_I32C(rowidx);
  TORCH_CHECK(h.dim() == 2 && h.is_contiguous() && rows.dim() == 2 && rows.is_contiguous() && out.is_contiguous());
  const int T = h.size(0), W = h.size(1), top = rowidx.size(1);
  TORCH_CHECK(rows.size(1) == W && out.numel() == h.numel() && rowidx.dim() == 2 && rowidx.size(0) == T);
  const bool weighted = w.numel() > 0;
  if (weighted) { CHECK_F32C(w); TORCH_CHECK(w.numel() == rowidx.numel()); }
  const bool ex = extra.numel() > 0;
  if (ex) {
    CHECK_ACT(extra); CHECK_SAME(extra, out); CHECK_ACT(extra_gate); CHECK_SAME(extra_gate, out);
    TORCH_CHECK(extra.is_contiguous() && extra.dim() == 2 && extra.size(0) == T && extra.size(1) == W);
    TORCH_CHECK(extra_gate.dim() == 1 && extra_gate.size(0) == T);
  }
  if (T == 0) return;
  seq_launch_moe_combine(out.data_ptr(), rows.data_ptr(), h.data_ptr(), rowidx.data_ptr<int>(),
                         weighted ? w.data_ptr<float>() : nullptr, ex ? extra.data_ptr() : nullptr,
                         ex ? extra_gate.data_ptr() : nullptr, ex ? (int)extra_gate.stride(0) : 0, T, W, top,
                         f32flag(out), cur_stream());
}

void wkv_recurrence(torch::Tensor o, torch::Tensor r, torch::Tensor k, torch::Tensor v, torch::Tensor d,
                    torch::Tensor w0, torch::Tensor u, torch::Tensor state, torch::Tensor slots, torch::Tensor cu,
                    torch::Tensor seg_start) {
  CHECK_F32C(o); CHECK_ACT(r); CHECK_ROWS3(r); CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_SAME(k, r); CHECK_SAME(v, r);
  CHECK_F32C(d); CHECK_F32C(w0); CHECK_F32C(u); CHECK_F32C(state);
  TORCH_CHECK(k.is_cuda() && v.is_cuda());
  const int T = r.size(0), H = r.size(1), D = r.size(2), V = v.size(2), B = slots.numel();
  check_segments(slots, cu, seg_start, T);
  TORCH_CHECK(k.size(0) == T && k.size(1) == H && k.size(2) == D && v.size(0) == T && v.size(1) == H);
  TORCH_CHECK(D <= 256, "the recurrence keeps up to 256 state rows per head in registers");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D && state.size(3) == V);
  TORCH_CHECK(d.numel() == (int64_t)T * H * D && w0.numel() == (int64_t)H * D && u.numel() == (int64_t)H * D &&
              o.numel() == (int64_t)T * H * V);
  if (T == 0 || B == 0) return;
  auto f32 = torch::dtype(torch::kFloat).device(r.device());
  auto rp = torch::empty({(int64_t)T, (int64_t)H * D}, f32), kp = torch::empty({(int64_t)T, (int64_t)H * D}, f32);
  auto wp = torch::empty({(int64_t)T, (int64_t)H * D}, f32), vp = torch::empty({(int64_t)T, (int64_t)H * V}, f32);
  auto bonus = torch::empty({(int64_t)T, (int64_t)H}, f32);
  seq_launch_wkv_recurrence(o.data_ptr<float>(), r.data_ptr(), k.data_ptr(), v.data_ptr(), d.data_ptr<float>(),
                            w0.data_ptr<float>(), u.data_ptr<float>(), rp.data_ptr<float>(), kp.data_ptr<float>(),
                            wp.data_ptr<float>(), vp.data_ptr<float>(), bonus.data_ptr<float>(),
                            state.data_ptr<float>(), slots.data_ptr<int>(), cu.data_ptr<int>(),
                            seg_start.data_ptr<int>(), T, B, H, D, V, (int)r.stride(0), (int)k.stride(0),
                            (int)v.stride(0), f32flag(r), cur_stream());
}

// state [slots, H, D+1, V+1]: the matrix, the normaliser as column V, the running maximum in row D
// o [T, H, V]: the read-out. With o empty, oe [T, H, V+1] (un-normalised read-out and normaliser) and
// mt [T, H] (running maxima) are filled instead, for a norm kernel that divides on the way.
void mlstm_recurrence(torch::Tensor o, torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor z,
                      torch::Tensor zb, double cap, torch::Tensor state, torch::Tensor slots, torch::Tensor cu,
                      torch::Tensor seg_start, torch::Tensor oe, torch::Tensor mt) {
  const bool raw = o.numel() == 0;
  if (!raw) { CHECK_F32C(o); }
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_SAME(k, q); CHECK_SAME(v, q);
  CHECK_F32C(z); CHECK_F32C(zb); CHECK_F32C(state);
  TORCH_CHECK(k.is_cuda() && v.is_cuda());
  const int T = q.size(0), H = q.size(1), D = q.size(2), V = v.size(2), B = slots.numel();
  check_segments(slots, cu, seg_start, T);
  TORCH_CHECK(k.size(0) == T && k.size(1) == H && k.size(2) == D && v.size(0) == T && v.size(1) == H);
  TORCH_CHECK(D <= 256, "the recurrence keeps up to 256 state rows per head in registers");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == D + 1 && state.size(3) == V + 1);
  TORCH_CHECK(z.numel() == (int64_t)T * 2 * H && zb.numel() == 2 * H && cap > 0);
  TORCH_CHECK(raw || o.numel() == (int64_t)T * H * V);
  auto f32 = torch::dtype(torch::kFloat).device(q.device());
  if (raw) {
    CHECK_F32C(oe); CHECK_F32C(mt);
    TORCH_CHECK(oe.numel() == (int64_t)T * H * (V + 1) && mt.numel() == (int64_t)T * H);
  } else {
    oe = torch::empty({(int64_t)T, (int64_t)H * (V + 1)}, f32);
    mt = torch::empty({(int64_t)T, (int64_t)H}, f32);
  }
  if (T == 0 || B == 0) return;
  auto qp = torch::empty({(int64_t)T, (int64_t)H * D}, f32), kp = torch::empty({(int64_t)T, (int64_t)H * D}, f32);
  auto vp = torch::empty({(int64_t)T, (int64_t)H * V}, f32);
  auto ig = torch::empty({(int64_t)T, (int64_t)H}, f32), fg = torch::empty({(int64_t)T, (int64_t)H}, f32);
  seq_launch_mlstm_recurrence(raw ? nullptr : o.data_ptr<float>(), q.data_ptr(), k.data_ptr(), v.data_ptr(), z.data_ptr<float>(),
                              zb.data_ptr<float>(), (float)cap, qp.data_ptr<float>(), kp.data_ptr<float>(),
                              vp.data_ptr<float>(), ig.data_ptr<float>(), fg.data_ptr<float>(),
                              oe.data_ptr<float>(), mt.data_ptr<float>(), state.data_ptr<float>(),
                              slots.data_ptr<int>(), cu.data_ptr<int>(), seg_start.data_ptr<int>(), T, B, H, D, V,
                              (int)q.stride(0), (int)k.stride(0), (int)v.stride(0), f32flag(q), cur_stream());
}

// ---- layer-normed sublayers with an input convolution, depth-weighted stream ----

// a / w_post empty: x_out = x_in. streams empty: no depth average.
void ln_residual_mix(torch::Tensor x_out, torch::Tensor x_in, torch::Tensor a, torch::Tensor w_post,
                     torch::Tensor stats, torch::Tensor streams, torch::Tensor dwa, int64_t n_prev, double eps) {
  CHECK_F32C(x_out); CHECK_F32C(x_in); CHECK_F32C(stats);
  TORCH_CHECK(x_in.dim() == 2 && x_out.sizes() == x_in.sizes());
  const int T = x_in.size(0), W = x_in.size(1);
  TORCH_CHECK(W >= 1 && W <= 16384 && stats.numel() == 2 * (int64_t)T);
  const bool has_a = a.numel() > 0, mix = streams.numel() > 0;
  if (has_a) {
    CHECK_ACT(a); CHECK_F32C(w_post);
    TORCH_CHECK(a.is_contiguous() && a.dim() == 2 && a.size(0) == T && a.size(1) == W && w_post.numel() == W);
  }
  if (mix) {
    CHECK_F32C(streams); CHECK_F32C(dwa);
    TORCH_CHECK(streams.dim() == 3 && streams.size(1) == T && streams.size(2) == W && n_prev >= 0 &&
                n_prev < streams.size(0) && dwa.numel() == n_prev + 1);
  }
  if (T == 0) return;
  seq_launch_ln_residual_mix(x_out.data_ptr<float>(), x_in.data_ptr<float>(), has_a ? a.data_ptr() : nullptr,
                             has_a ? w_post.data_ptr<float>() : nullptr, stats.data_ptr<float>(),
                             mix ? streams.data_ptr<float>() : nullptr, mix ? dwa.data_ptr<float>() : nullptr,
                             (int)n_prev, (int64_t)T * W, T, W, (float)eps, has_a ? f32flag(a) : 1, cur_stream());
}

// cw empty: the norm alone. hist: [slots, K-1, W] fp32 view (rows packed, free slot stride).
void ln_canon(torch::Tensor out, torch::Tensor x, torch::Tensor stats, torch::Tensor w, torch::Tensor cw,
              torch::Tensor hist, torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start,
              torch::Tensor token_seg) {
  CHECK_ACT(out); CHECK_F32C(x); CHECK_F32C(stats); CHECK_F32C(w);
  TORCH_CHECK(x.dim() == 2 && out.is_contiguous() && out.numel() == x.numel());
  const int T = x.size(0), W = x.size(1);
  TORCH_CHECK(w.numel() == W && stats.numel() == 2 * (int64_t)T);
  int K = 0, B = 0;
  int64_t hist_stride = 0;
  if (cw.numel() > 0) {
    CHECK_F32C(cw); CHECK_I32C(token_seg);
    check_segments(slots, cu, seg_start, T);
    TORCH_CHECK(cw.dim() == 2 && cw.size(1) == W && token_seg.numel() == T);
    K = cw.size(0);
    B = slots.numel();
    TORCH_CHECK(K >= 1 && K <= 16, "1..16 convolution taps supported");
    if (K > 1) {
      TORCH_CHECK(hist.is_cuda() && hist.scalar_type() == at::kFloat && hist.dim() == 3 && hist.size(1) == K - 1 &&
                  hist.size(2) == W && hist.stride(2) == 1 && hist.stride(1) == W);
      hist_stride = hist.stride(0);
    }
  }
  if (T == 0) return;
  seq_launch_ln_canon(out.data_ptr(), x.data_ptr<float>(), stats.data_ptr<float>(), w.data_ptr<float>(),
                      K ? cw.data_ptr<float>() : nullptr, K > 1 ? hist.data_ptr<float>() : nullptr, hist_stride,
                      K ? slots.data_ptr<int>() : nullptr, K ? cu.data_ptr<int>() : nullptr,
                      K ? seg_start.data_ptr<int>() : nullptr, K ? token_seg.data_ptr<int>() : nullptr, T, B, W, K,
                      f32flag(out), cur_stream());
}

// k empty: the layer reads another layer's cache, only q is normed and rotated
void qk_fullnorm_rope_store(torch::Tensor q, torch::Tensor k, torch::Tensor v, torch::Tensor wq, torch::Tensor wk,
                            double eps, torch::Tensor positions, torch::Tensor inv_freq, torch::Tensor k_cache,
                            torch::Tensor v_cache, torch::Tensor slots) {
  CHECK_ACT(q); CHECK_ROWS3(q); CHECK_F32C(wq); CHECK_I64C(positions); CHECK_F32C(inv_freq);
  const int T = q.size(0), H = q.size(1), D = q.size(2), R = inv_freq.numel();
  TORCH_CHECK(wq.numel() == (int64_t)H * D && positions.numel() == T && 2 * R <= D);
  const bool has_k = k.numel() > 0;
  int G = 0, Dv = 0, BS = 1;
  if (has_k) {
    CHECK_ROWS3(k); CHECK_ROWS3(v); CHECK_SAME(k, q); CHECK_SAME(v, q); CHECK_SAME(k_cache, q);
    CHECK_SAME(v_cache, q); CHECK_F32C(wk); CHECK_I64C(slots);
    TORCH_CHECK(k.is_cuda() && v.is_cuda() && k_cache.is_cuda() && v_cache.is_cuda() && k_cache.is_contiguous() &&
                v_cache.is_contiguous() && k_cache.dim() == 4 && v_cache.dim() == 4);
    G = k.size(1); Dv = v.size(2); BS = k_cache.size(2);
    TORCH_CHECK(k.size(0) == T && k.size(2) == D && v.size(0) == T && v.size(1) == G);
    TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D && v_cache.size(1) == G && v_cache.size(2) == BS &&
                v_cache.size(3) == Dv && v_cache.size(0) == k_cache.size(0));
    TORCH_CHECK(wk.numel() == (int64_t)G * D && slots.numel() == T);
  }
  TORCH_CHECK((int64_t)(H > G ? H : G) * D <= 15360, "projection too wide for the norm kernel's staging");
  if (T == 0) return;
  seq_launch_qk_fullnorm_rope_store(q.data_ptr(), has_k ? k.data_ptr() : nullptr, has_k ? v.data_ptr() : nullptr,
                                    wq.data_ptr<float>(), has_k ? wk.data_ptr<float>() : nullptr, (float)eps,
                                    positions.data_ptr<int64_t>(), inv_freq.data_ptr<float>(),
                                    has_k ? k_cache.data_ptr() : nullptr, has_k ? v_cache.data_ptr() : nullptr,
                                    has_k ? slots.data_ptr<int64_t>() : nullptr, T, H, G, D, Dv, R, BS,
                                    (int)q.stride(0), has_k ? (int)k.stride(0) : 0, has_k ? (int)v.stride(0) : 0,
                                    f32flag(q), cur_stream());
}

void pool_kv_update(torch::Tensor k_cache, torch::Tensor v_cache, torch::Tensor pool_k, torch::Tensor pool_v,
                    torch::Tensor block_tables, torch::Tensor token_seg, torch::Tensor positions, int64_t run,
                    torch::Tensor row_map) {
  CHECK_ACT(k_cache); CHECK_SAME(v_cache, k_cache); CHECK_F32C(pool_k); CHECK_F32C(pool_v);
  CHECK_I32C(block_tables); CHECK_I32C(token_seg); CHECK_I64C(positions);
  TORCH_CHECK(v_cache.is_cuda() && k_cache.is_contiguous() && v_cache.is_contiguous() && k_cache.dim() == 4 &&
              v_cache.dim() == 4 && pool_k.dim() == 4 && pool_v.dim() == 4 && block_tables.dim() == 2 && run >= 1);
  const int G = k_cache.size(1), BS = k_cache.size(2), D = k_cache.size(3), Dv = v_cache.size(3);
  const int PB = (BS + (int)run - 1) / (int)run;
  // row_map: the rows (of this step) to look at; empty = all
  const bool mapped = row_map.numel() > 0;
  if (mapped) { CHECK_I32C(row_map); TORCH_CHECK(row_map.numel() <= positions.numel()); }
  TORCH_CHECK(token_seg.numel() == positions.numel());
  const int T = mapped ? (int)row_map.numel() : (int)positions.numel();
  TORCH_CHECK(v_cache.size(0) == k_cache.size(0) && v_cache.size(1) == G && v_cache.size(2) == BS);
  TORCH_CHECK(pool_k.size(0) == k_cache.size(0) && pool_v.size(0) == k_cache.size(0) && pool_k.size(1) == G &&
              pool_v.size(1) == G && pool_k.size(2) == PB && pool_v.size(2) == PB && pool_k.size(3) == D &&
              pool_v.size(3) == Dv);
  if (T == 0) return;
  seq_launch_pool_kv_update(k_cache.data_ptr(), v_cache.data_ptr(), pool_k.data_ptr<float>(),
                            pool_v.data_ptr<float>(), block_tables.data_ptr<int>(), token_seg.data_ptr<int>(),
                            positions.data_ptr<int64_t>(), mapped ? row_map.data_ptr<int>() : nullptr, (int)run, PB,
                            T, G, D, Dv, BS,
                            (int)block_tables.stride(0), f32flag(k_cache), cur_stream());
}

// x [T, H, V], B / C [T, G, N] row views, dt [T, H] row view; state [slots, H, N, V] fp32
void ssd_recurrence(torch::Tensor o, torch::Tensor x, torch::Tensor Bm, torch::Tensor Cm, torch::Tensor dt,
                    torch::Tensor dt_bias, torch::Tensor a_log, torch::Tensor skip, torch::Tensor state,
                    torch::Tensor slots, torch::Tensor cu, torch::Tensor seg_start) {
  CHECK_F32C(o); CHECK_ACT(x); CHECK_ROWS3(x); CHECK_ROWS3(Bm); CHECK_ROWS3(Cm); CHECK_ROWS2(dt);
  CHECK_SAME(Bm, x); CHECK_SAME(Cm, x); CHECK_SAME(dt, x);
  CHECK_F32C(dt_bias); CHECK_F32C(a_log); CHECK_F32C(skip); CHECK_F32C(state);
  check_segments(slots, cu, seg_start, state);
  const int T = x.size(0), H = x.size(1), V = x.size(2), G = Bm.size(1), N = Bm.size(2), B = slots.numel();
  TORCH_CHECK(Bm.is_cuda() && Cm.is_cuda() && dt.is_cuda() && Bm.size(0) == T && Cm.size(0) == T &&
              Cm.size(1) == G && Cm.size(2) == N && dt.size(0) == T && dt.size(1) == H && G >= 1 && H % G == 0);
  TORCH_CHECK(N <= 256, "state size above 256 is not supported by the recurrence kernel");
  TORCH_CHECK(state.dim() == 4 && state.size(1) == H && state.size(2) == N && state.size(3) == V);
  TORCH_CHECK(dt_bias.numel() == H && a_log.numel() == H && skip.numel() == H && o.numel() == (int64_t)T * H * V);
  if (T == 0 || B == 0) return;
  auto opt = torch::dtype(torch::kFloat).device(x.device());
  auto packed = torch::empty({(int64_t)T, (int64_t)H * (2 * N + V)}, opt);
  auto dec = torch::empty({(int64_t)T, (int64_t)H}, opt);
  seq_launch_ssd_recurrence(o.data_ptr<float>(), x.data_ptr(), Bm.data_ptr(), Cm.data_ptr(), dt.data_ptr(),
                            dt_bias.data_ptr<float>(), a_log.data_ptr<float>(), skip.data_ptr<float>(),
                            packed.data_ptr<float>(), dec.data_ptr<float>(), state.data_ptr<float>(),
                            slots.data_ptr<int>(), cu.data_ptr<int>(), seg_start.data_ptr<int>(), T, B, H, G, N, V,
                            (int)x.stride(0), (int)Bm.stride(0), (int)Cm.stride(0), (int)dt.stride(0), f32flag(x),
                            cur_stream());
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  m.def("embed_rmsnorm", &embed_rmsnorm);
  m.def("rmsnorm_cast", &rmsnorm_cast);
  m.def("sandwich_residual", &sandwich_residual);
  m.def("gated_rmsnorm", &gated_rmsnorm);
  m.def("gated_act", &gated_act);
  m.def("rope_pairs_store", &rope_pairs_store);
  m.def("attn_masked_paged", &attn_masked_paged);
  m.def("qk_norm_store", &qk_norm_store);
  m.def("embed_bigram", &embed_bigram);
  m.def("group_norm_pair", &group_norm_pair);
  m.def("cast_concat", &cast_concat);
  m.def("head_rmsnorm_gate", &head_rmsnorm_gate);
  m.def("token_shift_mix", &token_shift_mix);
  m.def("moe_route", &moe_route);
  m.def("moe_combine", &moe_combine);
  m.def("gelu_tanh", &gelu_tanh);
  m.def("scale_softcap", &scale_softcap);
  m.def("scale_rows", &scale_rows);
  m.def("moe_spread_rows", &moe_spread_rows);
  m.def("latent_kv_store", &latent_kv_store);
  m.def("attn_latent_paged", &attn_latent_paged);
  m.def("wkv_recurrence", &wkv_recurrence);
  m.def("mlstm_recurrence", &mlstm_recurrence);
  m.def("head_gate", &head_gate);
  m.def("attn_varlen_mfma", &attn_varlen_mfma);
  m.def("linear_attn_decay", &linear_attn_decay);
  m.def("causal_conv_silu", &causal_conv_silu);
  m.def("gated_delta_rule", &gated_delta_rule);
  m.def("ln_residual_mix", &ln_residual_mix);
  m.def("ln_canon", &ln_canon);
  m.def("qk_fullnorm_rope_store", &qk_fullnorm_rope_store);
  m.def("pool_kv_update", &pool_kv_update);
  m.def("ssd_recurrence", &ssd_recurrence);
}
