// Recurrent sequence mixers over segments: decayed linear attention, short
// causal convolution with carried taps, and the gated delta rule with a decay
// per key channel. State lives in fp32 slots [slot, H, D, V]; a segment that
// starts a sequence (seg_start == 0) takes its state as zero whatever the
// slot holds, so a reused slot needs no clearing.
//
// Layout of the recurrences: one wave per (segment, head, 32 state columns).
// The two half-waves split the state's rows: lane (half, j) keeps rows
// half*D/2 .. of column j in registers, so the per-token update is lane-local
// and the read-out needs one exchange between the halves; slot traffic is
// coalesced over j. Splitting columns and rows over many small waves keeps a
// few long prompts from running on a handful of SIMDs.

#include "seq_common.h"

// ---- decayed linear attention ------------------------------------------------
// S <- decay_h S + silu(k) silu(v)^T ; o = S^T silu(q)
//
// Two kernels. A parallel pre-pass applies silu and packs q|k|v per (token,
// head) in fp32; the recurrence then only loads and multiplies. One wave of
// the recurrence serves (segment, head, 64/NS state columns): its NS lane
// groups split the state's rows (DMAX/NS each, in registers), so the update is
// lane-local and the read-out is reduced over the groups with NS-1 exchanges.
// A single wave issues slowly on this hardware; NS is chosen at launch so that
// there are several waves per SIMD even for a few long prompts.
template <typename T>
__global__ void linear_prep_kernel(float* __restrict__ pk, const T* __restrict__ q,
                                   const T* __restrict__ k, const T* __restrict__ v, int64_t n, int H,
                                   int D, int V, int q_stride, int k_stride, int v_stride) {
  const int W = 2 * D + V;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / W;
    const int c = (int)(i - th * W);
    const int64_t t = th / H;
    const int h = (int)(th - t * H);
    float x;
    if (c < D) x = ldf(q + t * q_stride + (int64_t)h * D + c);
    else if (c < 2 * D) x = ldf(k + t * k_stride + (int64_t)h * D + (c - D));
    else x = ldf(v + t * v_stride + (int64_t)h * V + (c - 2 * D));
    pk[i] = silu_exact(x);
  }
}

// 8-wide form: D, V and the strides are multiples of 8, so a group of 8
// never straddles q | k | v
template <typename T>
__global__ void linear_prep_v8_kernel(float* __restrict__ pk, const T* __restrict__ q,
                                      const T* __restrict__ k, const T* __restrict__ v, int64_t n8, int H,
                                      int D, int V, int q_stride, int k_stride, int v_stride) {
  const int W8 = (2 * D + V) / 8;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / W8;
    const int c = (int)(i - th * W8) * 8;
    const int64_t t = th / H;
    const int h = (int)(th - t * H);
    float x[8];
    if (c < D) ld8(q + t * q_stride + (int64_t)h * D + c, x);
    else if (c < 2 * D) ld8(k + t * k_stride + (int64_t)h * D + (c - D), x);
    else ld8(v + t * v_stride + (int64_t)h * V + (c - 2 * D), x);
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = silu_exact(x[e]);
    st8(pk + i * 8, x);
  }
}

template <int DMAX, int NS>
__global__ void __launch_bounds__(WAVE) linear_attn_decay_kernel(
    float* __restrict__ o, const float* __restrict__ pk, const float* __restrict__ decay,
    const float* __restrict__ decay_t, const float* __restrict__ skip,
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ cu,
    const int* __restrict__ seg_start, int H, int D, int V) {
  // decay_t != nullptr: one decay per (token, head) [T, H] instead of decay[h];
  // skip != nullptr: o += skip[h] * v (a direct path from the value to the output)
  constexpr int TB = 4;                                   // tokens per pipeline stage
  constexpr int DR = DMAX / NS, COLS = WAVE / NS;         // state rows / columns per lane group
  constexpr int PER = (2 * DMAX + WAVE - 1) / WAVE;       // q|k elements staged per lane
  __shared__ float qk[2][TB][2 * DMAX];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int grp = lane / COLS, j = blockIdx.z * COLS + (lane % COLS), d0 = grp * DR;
  const bool live = j < V;
  const int t0 = cu[b], t1 = cu[b + 1];
  const int W = 2 * D + V;
  float* sp = state + (((int64_t)slots[b] * H + h) * D) * V + j;
  float S[DR];
  const bool fresh = seg_start[b] == 0;
#pragma unroll
  for (int d = 0; d < DR; ++d) S[d] = (!fresh && live && d0 + d < D) ? sp[(int64_t)(d0 + d) * V] : 0.f;
  const float dec = decay_t ? 0.f : decay[h];
  const float skp = skip ? skip[h] : 0.f;
  if (t1 - t0 == 1) {
    // decode: one row. No pipeline — stage q|k once (zeros above D), update, read out.
    const float* row = pk + ((int64_t)t0 * H + h) * W;
    float* buf = qk[0][0];
    for (int i = lane; i < 2 * DMAX; i += WAVE) {
      const int d = i < DMAX ? i : i - DMAX;
      buf[i] = d < D ? row[i < DMAX ? d : D + d] : 0.f;
    }
    const float vj = live ? row[2 * D + j] : 0.f;
    const float dc = decay_t ? decay_t[(int64_t)t0 * H + h] : dec;
    __syncthreads();
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < DR; ++d) {
      S[d] = dc * S[d] + buf[DMAX + d0 + d] * vj;
      acc += S[d] * buf[d0 + d];
    }
#pragma unroll
    for (int off = COLS; off < WAVE; off <<= 1) acc += __shfl_xor(acc, off);
    if (live) {
      if (grp == 0) o[((int64_t)t0 * H + h) * V + j] = acc + skp * vj;
#pragma unroll
      for (int d = 0; d < DR; ++d) if (d0 + d < D) sp[(int64_t)(d0 + d) * V] = S[d];
    }
    return;
  }
  // rows D..DMAX-1 of the staging buffers stay zero, so the unrolled loops
  // below run over DMAX without a bound check (a branch per row would keep
  // the LDS reads from being batched)
  for (int i = lane; i < 2 * TB * 2 * DMAX; i += WAVE) (&qk[0][0][0])[i] = 0.f;
  __syncthreads();
  // software pipeline over groups of TB tokens: the next group's operands are
  // in flight while this group's tokens are computed one after the other
  float pre[TB][PER], vpre[TB], dpre[TB];
  auto fetch = [&](int tg) {
#pragma unroll
    for (int u = 0; u < TB; ++u) {
      const int t = tg + u;
      const bool on = t < t1;
      const float* row = pk + ((int64_t)t * H + h) * W;
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        const int i = lane + r * WAVE;
        pre[u][r] = (on && i < 2 * D) ? row[i] : 0.f;
      }
      vpre[u] = (on && live) ? row[2 * D + j] : 0.f;
      dpre[u] = (on && decay_t) ? decay_t[(int64_t)t * H + h] : dec;
    }
  };
  if (t0 < t1) fetch(t0);
  int flip = 0;
  for (int tg = t0; tg < t1; tg += TB, flip ^= 1) {
    float vj[TB], dc[TB];
#pragma unroll
    for (int u = 0; u < TB; ++u) {
#pragma unroll
      for (int r = 0; r < PER; ++r) {
        const int i = lane + r * WAVE;
        if (i < 2 * D) qk[flip][u][i < D ? i : DMAX + (i - D)] = pre[u][r];
      }
      vj[u] = vpre[u];
      dc[u] = dpre[u];
    }
    __syncthreads();    // double-buffered: one barrier per group
    if (tg + TB < t1) fetch(tg + TB);
#pragma unroll
    for (int u = 0; u < TB; ++u) {
      if (tg + u < t1) {
        const float* buf = qk[flip][u];
        float acc = 0.f;
#pragma unroll
        for (int d = 0; d < DR; ++d) {
          S[d] = dc[u] * S[d] + buf[DMAX + d0 + d] * vj[u];
          acc += S[d] * buf[d0 + d];
        }
#pragma unroll
        for (int off = COLS; off < WAVE; off <<= 1) acc += __shfl_xor(acc, off);
        if (live && grp == 0) o[((int64_t)(tg + u) * H + h) * V + j] = acc + skp * vj[u];
      }
    }
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DR; ++d) if (d0 + d < D) sp[(int64_t)(d0 + d) * V] = S[d];
  }
}

// ---- short causal convolution + silu ----------------------------------------
// y[t,c] = silu(bias[c] + sum_j w[j,c] * x[t - (K-1-j), c]) (bias optional; weights taps-major [K, C],
// last tap = current token); inputs before the segment
// come from conv_state [slot, K-1, C] (oldest first), zeros for a fresh sequence.
template <typename T>
__global__ void causal_conv_silu_kernel(T* __restrict__ y, const T* __restrict__ x,
                                        const float* __restrict__ w, const T* __restrict__ conv_state,
                                        const int* __restrict__ slots, const int* __restrict__ cu,
                                        const int* __restrict__ seg_start, const int* __restrict__ token_seg,
                                        const float* __restrict__ bias, int64_t n, int C, int K, int x_stride) {
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int t = (int)(idx / C), c = (int)(idx - (int64_t)t * C);
    const int b = token_seg[t];
    const int i = t - cu[b];
    const bool fresh = seg_start[b] == 0;
    const T* hist = conv_state + (int64_t)slots[b] * (K - 1) * C;
    float acc = bias ? bias[c] : 0.f;
    for (int j = 0; j < K; ++j) {
      const int src = i - (K - 1 - j);
      float xv;
      if (src >= 0) xv = ldf(x + (int64_t)(t - (K - 1 - j)) * x_stride + c);
      else xv = fresh ? 0.f : ldf(hist + (int64_t)(K - 1 + src) * C + c);
      acc += w[(int64_t)j * C + c] * xv;
    }
    stf(y + idx, silu_exact(acc));
  }
}

// 8 channels per thread (C and the row stride multiples of 8)
template <typename T>
__global__ void causal_conv_silu_v8_kernel(T* __restrict__ y, const T* __restrict__ x,
                                           const float* __restrict__ w, const T* __restrict__ conv_state,
                                           const int* __restrict__ slots, const int* __restrict__ cu,
                                           const int* __restrict__ seg_start,
                                           const int* __restrict__ token_seg,
                                           const float* __restrict__ bias, int64_t n8, int C, int K,
                                           int x_stride) {
  const int C8 = C / 8;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n8;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int t = (int)(idx / C8), c = (int)(idx - (int64_t)t * C8) * 8;
    const int b = token_seg[t];
    const int i = t - cu[b];
    const bool fresh = seg_start[b] == 0;
    const T* hist = conv_state + (int64_t)slots[b] * (K - 1) * C;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (bias) ld8(bias + c, acc);
    for (int j = 0; j < K; ++j) {
      const int src = i - (K - 1 - j);
      float xv[8], wv[8];
      if (src >= 0) ld8(x + (int64_t)(t - (K - 1 - j)) * x_stride + c, xv);
      else if (!fresh) ld8(hist + (int64_t)(K - 1 + src) * C + c, xv);
      else continue;
      ld8(w + (int64_t)j * C + c, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += wv[e] * xv[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = silu_exact(acc[e]);
    st8(y + (int64_t)t * C + c, acc);
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
// Pre-pass, parallel over tokens — one wave per (token, q/k head) and one per
// (token, value head):
//   qn = q / sqrt(|q|^2 + 1e-6) * D^-1/2,  kn = k / sqrt(|k|^2 + 1e-6)     [T, G, D] fp32
//   g  = exp(-exp(A_h) softplus(a + dt))                                    [T, H, D] fp32
//   vf = v, beta = sigmoid(b)                                              [T, H, V], [T, H] fp32
template <typename T>
__global__ void delta_prep_kernel(float* __restrict__ qn, float* __restrict__ kn, float* __restrict__ gd,
                                  float* __restrict__ vf, float* __restrict__ bt, const T* __restrict__ q,
                                  const T* __restrict__ k, const T* __restrict__ v,
                                  const T* __restrict__ beta_logit, const T* __restrict__ a,
                                  const float* __restrict__ dt_bias, const float* __restrict__ a_log,
                                  int H, int G, int D, int V, int q_stride, int k_stride, int v_stride,
                                  int beta_stride, int a_stride) {
  const int64_t t = blockIdx.x;
  const int y = blockIdx.y, lane = threadIdx.x;
  if (y < G) {
    const T* qr = q + t * q_stride + (int64_t)y * D;
    const T* kr = k + t * k_stride + (int64_t)y * D;
    float sq = 0.f, sk = 0.f;
    for (int d = lane; d < D; d += WAVE) {
      const float x = ldf(qr + d), z = ldf(kr + d);
      sq += x * x; sk += z * z;
    }
    sq = wave_sum(sq); sk = wave_sum(sk);
    const float rq = 1.0f / (sqrtf(sq + 1e-6f) * sqrtf((float)D)), rk = 1.0f / sqrtf(sk + 1e-6f);
    for (int d = lane; d < D; d += WAVE) {
      qn[(t * G + y) * D + d] = ldf(qr + d) * rq;
      kn[(t * G + y) * D + d] = ldf(kr + d) * rk;
    }
  } else {
    const int h = y - G;
    const float rate = expf(a_log[h]);
    for (int d = lane; d < D; d += WAVE) {
      const float pre = ldf(a + t * a_stride + (int64_t)h * D + d) + dt_bias[(int64_t)h * D + d];
      gd[(t * H + h) * D + d] = expf(-rate * softplus_exact(pre));
    }
    for (int i = lane; i < V; i += WAVE) vf[(t * H + h) * V + i] = ldf(v + t * v_stride + (int64_t)h * V + i);
    if (lane == 0) bt[t * H + h] = sigmoid_exact(ldf(beta_logit + t * beta_stride + h));
  }
}

// The recurrence proper, on the pre-pass's fp32 operands; wave layout and
// pipeline as in linear_attn_decay_kernel.
template <int DMAX, int NS>
__global__ void __launch_bounds__(WAVE) gated_delta_rule_kernel(
    float* __restrict__ o, const float* __restrict__ qn, const float* __restrict__ kn,
    const float* __restrict__ gd, const float* __restrict__ vf, const float* __restrict__ bt,
    float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ cu,
    const int* __restrict__ seg_start, int H, int G, int D, int V) {
  constexpr int TB = 4;
  constexpr int DR = DMAX / NS, COLS = WAVE / NS;
  constexpr int PER = (3 * DMAX + WAVE - 1) / WAVE;       // q|k|g elements staged per lane
  __shared__ float buf_[2][TB][3 * DMAX];
  const int b = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int grp = lane / COLS, j = blockIdx.z * COLS + (lane % COLS), d0 = grp * DR;
  const int g = h / (H / G);
  const bool live = j < V;
  const int t0 = cu[b], t1 = cu[b + 1];
  float* sp = state + (((int64_t)slots[b] * H + h) * D) * V + j;
  float S[DR];
  const bool fresh = seg_start[b] == 0;
#pragma unroll
  for (int d = 0; d < DR; ++d) S[d] = (!fresh && live && d0 + d < D) ? sp[(int64_t)(d0 + d) * V] : 0.f;
  if (t1 - t0 == 1) {
    // decode: one row, no pipeline (see linear_attn_decay_kernel)
    float* buf = buf_[0][0];
    for (int i = lane; i < 3 * DMAX; i += WAVE) {
      const int which = i / DMAX, d = i - which * DMAX;
      float val = 0.f;
      if (d < D)
        val = which == 0 ? qn[((int64_t)t0 * G + g) * D + d]
            : which == 1 ? kn[((int64_t)t0 * G + g) * D + d] : gd[((int64_t)t0 * H + h) * D + d];
      buf[i] = val;
    }
    const float vj = live ? vf[((int64_t)t0 * H + h) * V + j] : 0.f;
    const float beta = bt[(int64_t)t0 * H + h];
    __syncthreads();
    float pred = 0.f;
#pragma unroll
    for (int d = 0; d < DR; ++d) {
      S[d] *= buf[2 * DMAX + d0 + d];
      pred += S[d] * buf[DMAX + d0 + d];
    }
#pragma unroll
    for (int off = COLS; off < WAVE; off <<= 1) pred += __shfl_xor(pred, off);
    const float uu = beta * (vj - pred);
    float acc = 0.f;
#pragma unroll
    for (int d = 0; d < DR; ++d) {
      S[d] += buf[DMAX + d0 + d] * uu;
      acc += S[d] * buf[d0 + d];
    }
#pragma unroll
    for (int off = COLS; off < WAVE; off <<= 1) acc += __shfl_xor(acc, off);
    if (live) {
      if (grp == 0) o[((int64_t)t0 * H + h) * V + j] = acc;
#pragma unroll
      for (int d = 0; d < DR; ++d) if (d0 + d < D) sp[(int64_t)(d0 + d) * V] = S[d];
    }
    return;
  }
  for (int i = lane; i < 2 * TB * 3 * DMAX; i += WAVE) (&buf_[0][0][0])[i] = 0.f;   // pad rows stay zero
  __syncthreads();
  float pre[TB][PER], vpre[TB], bpre[TB];
  // where each staged element comes from and goes to, fixed per lane: element
  // i = lane + r*64 of q|k|g (no index division inside the token loop)
  const float* src[PER];
  int src_step[PER], dst[PER];
#pragma unroll
  for (int r = 0; r < PER; ++r) {
    const int i = lane + r * WAVE;
    const int which = i / D, d = i - which * D;
    dst[r] = which < 3 ? which * DMAX + d : -1;
    src[r] = which == 0 ? qn + (int64_t)g * D + d : which == 1 ? kn + (int64_t)g * D + d : gd + (int64_t)h * D + d;
    src_step[r] = which == 2 ? H * D : G * D;
  }
  auto fetch = [&](int tg) {
#pragma unroll
    for (int u = 0; u < TB; ++u) {
      const int t = tg + u;
      const bool on = t < t1;
#pragma unroll
      for (int r = 0; r < PER; ++r) pre[u][r] = (on && dst[r] >= 0) ? src[r][(int64_t)t * src_step[r]] : 0.f;
      vpre[u] = (on && live) ? vf[((int64_t)t * H + h) * V + j] : 0.f;
      bpre[u] = on ? bt[(int64_t)t * H + h] : 0.f;
    }
  };
  if (t0 < t1) fetch(t0);
  int flip = 0;
  for (int tg = t0; tg < t1; tg += TB, flip ^= 1) {
    float vj[TB], beta[TB];
#pragma unroll
    for (int u = 0; u < TB; ++u) {
#pragma unroll
      for (int r = 0; r < PER; ++r)
        if (dst[r] >= 0) buf_[flip][u][dst[r]] = pre[u][r];
      vj[u] = vpre[u];
      beta[u] = bpre[u];
    }
    __syncthreads();
    if (tg + TB < t1) fetch(tg + TB);
#pragma unroll
    for (int u = 0; u < TB; ++u) {
      if (tg + u < t1) {
        const float* buf = buf_[flip][u];
        float pred = 0.f;
#pragma unroll
        for (int d = 0; d < DR; ++d) {
          S[d] *= buf[2 * DMAX + d0 + d];
          pred += S[d] * buf[DMAX + d0 + d];
        }
#pragma unroll
        for (int off = COLS; off < WAVE; off <<= 1) pred += __shfl_xor(pred, off);
        const float uu = beta[u] * (vj[u] - pred);
        float acc = 0.f;
#pragma unroll
        for (int d = 0; d < DR; ++d) {
          S[d] += buf[DMAX + d0 + d] * uu;
          acc += S[d] * buf[d0 + d];
        }
#pragma unroll
        for (int off = COLS; off < WAVE; off <<= 1) acc += __shfl_xor(acc, off);
        if (live && grp == 0) o[((int64_t)(tg + u) * H + h) * V + j] = acc;
      }
    }
  }
  if (live) {
#pragma unroll
    for (int d = 0; d < DR; ++d) if (d0 + d < D) sp[(int64_t)(d0 + d) * V] = S[d];
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

#define DISPATCH_D(D, ...)                                          \
  if (D <= 32) { constexpr int DMAX = 32; __VA_ARGS__ }             \
  else if (D <= 64) { constexpr int DMAX = 64; __VA_ARGS__ }        \
  else if (D <= 128) { constexpr int DMAX = 128; __VA_ARGS__ }      \
  else { constexpr int DMAX = 256; __VA_ARGS__ }

// rows of the state are split over NS lane groups; more groups = more, smaller
// waves with fewer registers each. Take the coarsest split that still gives
// every SIMD (1024 of them) many waves to switch between.
static inline int pick_split(int B, int H, int V) {
  const int64_t want = 16384;
  for (int ns = 2; ns <= 8; ns *= 2)
    if ((int64_t)B * H * ((V + 64 / ns - 1) / (64 / ns)) >= want) return ns;
  return 8;
}

#define DISPATCH_NS(ns, ...)                                        \
  if (ns == 2) { constexpr int NS = 2; __VA_ARGS__ }                \
  else if (ns == 4) { constexpr int NS = 4; __VA_ARGS__ }           \
  else { constexpr int NS = 8; __VA_ARGS__ }

extern "C" void seq_launch_linear_attn_decay(float* o, const void* q, const void* k, const void* v,
                                             const float* decay, float* packed, float* state,
                                             const int* slots, const int* cu, const int* seg_start, int T_,
                                             int B, int H, int D, int V, int q_stride, int k_stride,
                                             int v_stride, int is_f32, hipStream_t st) {
  const int64_t n = (int64_t)T_ * H * (2 * D + V);
  const int grid = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
  if (D % 8 == 0 && V % 8 == 0 && q_stride % 8 == 0 && k_stride % 8 == 0 && v_stride % 8 == 0 &&
      aligned16(q) && aligned16(k) && aligned16(v) && aligned16(packed)) {
    const int g8 = (int)((n / 8 + 255) / 256 < 16384 ? (n / 8 + 255) / 256 : 16384);
    DISPATCH_T(is_f32, hipLaunchKernelGGL(linear_prep_v8_kernel<T>, dim3(g8), dim3(256), 0, st, packed,
                                          (const T*)q, (const T*)k, (const T*)v, n / 8, H, D, V, q_stride,
                                          k_stride, v_stride);)
  } else {
    DISPATCH_T(is_f32, hipLaunchKernelGGL(linear_prep_kernel<T>, dim3(grid), dim3(256), 0, st, packed,
                                          (const T*)q, (const T*)k, (const T*)v, n, H, D, V, q_stride, k_stride,
                                          v_stride);)
  }
  const int ns = pick_split(B, H, V);
  DISPATCH_NS(ns, DISPATCH_D(D, hipLaunchKernelGGL((linear_attn_decay_kernel<DMAX, NS>),
                                                   dim3(B, H, (V + WAVE / NS - 1) / (WAVE / NS)), dim3(WAVE), 0,
                                                   st, o, packed, decay, nullptr, nullptr, state, slots, cu,
                                                   seg_start, H, D, V);))
}

// ---- state-space recurrence with a scalar decay per head and token ---------------
// d = softplus(dt + dt_bias); S <- exp(-exp(A_h) d) S + (d B_g) x_h^T; o = S^T C_g + D_h x_h
// A parallel pre-pass (one wave per (token, head)) writes the recurrence's
// operands in fp32 in the packed layout of linear_attn_decay_kernel —
// [C_g (N) | d B_g (N) | x_h (V)] — and the decay per (token, head); the
// recurrence itself is that kernel with a per-token decay and the skip term.
template <typename T>
__global__ void ssd_prep_kernel(float* __restrict__ pk, float* __restrict__ dec, const T* __restrict__ x,
                                const T* __restrict__ Bm, const T* __restrict__ Cm, const T* __restrict__ dt,
                                const float* __restrict__ dt_bias, const float* __restrict__ a_log, int H, int G,
                                int N, int V, int x_stride, int b_stride, int c_stride, int dt_stride) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  const float d = softplus_exact(ldf(dt + t * dt_stride + h) + dt_bias[h]);
  if (lane == 0) dec[t * H + h] = expf(-expf(a_log[h]) * d);
  float* row = pk + (t * H + h) * (2 * N + V);
  const T* cr = Cm + t * c_stride + (int64_t)g * N;
  const T* br = Bm + t * b_stride + (int64_t)g * N;
  const T* xr = x + t * x_stride + (int64_t)h * V;
  for (int i = lane; i < N; i += WAVE) { row[i] = ldf(cr + i); row[N + i] = d * ldf(br + i); }
  for (int i = lane; i < V; i += WAVE) row[2 * N + i] = ldf(xr + i);
}

extern "C" void seq_launch_ssd_recurrence(float* o, const void* x, const void* Bm, const void* Cm, const void* dt,
                                          const float* dt_bias, const float* a_log, const float* skip,
                                          float* packed, float* dec, float* state, const int* slots,
                                          const int* cu, const int* seg_start, int T_, int B, int H, int G, int N,
                                          int V, int x_stride, int b_stride, int c_stride, int dt_stride,
                                          int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(ssd_prep_kernel<T>, dim3(T_, H), dim3(WAVE), 0, st, packed, dec,
                                        (const T*)x, (const T*)Bm, (const T*)Cm, (const T*)dt, dt_bias, a_log, H,
                                        G, N, V, x_stride, b_stride, c_stride, dt_stride);)
  const int ns = pick_split(B, H, V);
  const int D = N;
  DISPATCH_NS(ns, DISPATCH_D(D, hipLaunchKernelGGL((linear_attn_decay_kernel<DMAX, NS>),
                                                   dim3(B, H, (V + WAVE / NS - 1) / (WAVE / NS)), dim3(WAVE), 0,
                                                   st, o, packed, nullptr, dec, skip, state, slots, cu, seg_start,
                                                   H, N, V);))
}

extern "C" void seq_launch_causal_conv_silu(void* y, const void* x, const float* w, void* conv_state,
                                            const int* slots, const int* cu, const int* seg_start,
                                            const int* token_seg, const float* bias, int T_, int B, int C, int K,
                                            int x_stride, int is_f32, hipStream_t st) {
  const int64_t n = (int64_t)T_ * C;
  const int grid = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  const int grid2 = (int)(((int64_t)B * C + 255) / 256);
  const bool v8 = C % 8 == 0 && x_stride % 8 == 0 && aligned16(y) && aligned16(x) && aligned16(conv_state) &&
                  aligned16(w) && (bias == nullptr || aligned16(bias));
  const int g8 = (int)((n / 8 + 255) / 256 < 16384 ? (n / 8 + 255) / 256 : 16384);
  DISPATCH_T(is_f32,
             if (v8) hipLaunchKernelGGL(causal_conv_silu_v8_kernel<T>, dim3(g8), dim3(256), 0, st, (T*)y,
                                        (const T*)x, w, (const T*)conv_state, slots, cu, seg_start, token_seg,
                                        bias, n / 8, C, K, x_stride);
             else hipLaunchKernelGGL(causal_conv_silu_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)y, (const T*)x,
                                w, (const T*)conv_state, slots, cu, seg_start, token_seg, bias, n, C, K, x_stride);
             if (K > 1) hipLaunchKernelGGL(conv_state_update_kernel<T>, dim3(grid2), dim3(256), 0, st, (const T*)x,
                                (T*)conv_state, slots, cu, seg_start, B, C, K, x_stride);)
}

extern "C" void seq_launch_gated_delta_rule(float* o, const void* q, const void* k, const void* v,
                                            const void* beta_logit, const void* a, const float* dt_bias,
                                            const float* a_log, float* qn, float* kn, float* gd, float* vf,
                                            float* bt, float* state, const int* slots, const int* cu,
                                            const int* seg_start, int T_, int B, int H, int G, int D, int V,
                                            int q_stride, int k_stride, int v_stride, int beta_stride,
                                            int a_stride, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(delta_prep_kernel<T>, dim3(T_, G + H), dim3(WAVE), 0, st, qn, kn, gd,
                                        vf, bt, (const T*)q, (const T*)k, (const T*)v, (const T*)beta_logit,
                                        (const T*)a, dt_bias, a_log, H, G, D, V, q_stride, k_stride, v_stride,
                                        beta_stride, a_stride);)
  const int ns = pick_split(B, H, V);
  DISPATCH_NS(ns, DISPATCH_D(D, hipLaunchKernelGGL((gated_delta_rule_kernel<DMAX, NS>),
                                                   dim3(B, H, (V + WAVE / NS - 1) / (WAVE / NS)), dim3(WAVE), 0,
                                                   st, o, qn, kn, gd, vf, bt, state, slots, cu, seg_start, H, G,
                                                   D, V);))
}
