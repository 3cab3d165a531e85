// Kernels of the parallel-layer family: hashed bigram embedding, the grouped
// RMS norm fused with the residual add of two branches, the loop-entry
// concatenation, per-head norm + gate after a recurrence, token shift, the
// expert router and the weighted gather that combines expert outputs.
// The residual stream, norms, router and gates are fp32; T is the activation
// type (bf16 when serving, fp32 in exact mode).

#include "seq_common.h"

// ---- embedding: table[id] * scale + bigram[hash(prev, id)] -------------------
// The previous token of a segment's first row is the sequence's carried token
// (tok_state[slot]); a sequence's very first token takes the table's last row.
template <typename T>
__global__ void embed_bigram_kernel(float* __restrict__ out, const int64_t* __restrict__ ids,
                                    const T* __restrict__ table, const T* __restrict__ bigram, float scale,
                                    int mul_prev, int mul_cur, int buckets, const int* __restrict__ tok_state,
                                    const int* __restrict__ slots, const int* __restrict__ cu,
                                    const int* __restrict__ seg_start, const int* __restrict__ token_seg, int W) {
  const int t = blockIdx.x;
  const int64_t id = ids[t];
  const T* erow = table + id * W;
  const T* brow = nullptr;
  if (bigram != nullptr) {
    const int b = token_seg[t];
    int64_t row;
    if (t == cu[b] && seg_start[b] == 0) {
      row = buckets;
    } else {
      const int64_t prev = t == cu[b] ? (int64_t)tok_state[slots[b]] : ids[t - 1];
      row = (prev * mul_prev + id * mul_cur) % buckets;
    }
    brow = bigram + row * W;
  }
  float* orow = out + (int64_t)t * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    orow[i] = ldf(erow + i) * scale + (brow ? ldf(brow + i) : 0.f);
}

// after the rows are embedded: the segment's last id becomes the carried token
__global__ void tok_state_update_kernel(const int64_t* __restrict__ ids, int* __restrict__ tok_state,
                                        const int* __restrict__ slots, const int* __restrict__ cu, int B) {
  const int b = blockIdx.x * blockDim.x + threadIdx.x;
  if (b >= B) return;
  if (cu[b + 1] > cu[b]) tok_state[slots[b]] = (int)ids[cu[b + 1] - 1];
}

// ---- residual add + grouped RMS norm under two weights ------------------------
// x += a + b (branches optional); n = x with each of `groups` equal runs divided
// by its own sqrt(mean square + eps); out1 = n * w1, out2 = n * w2 (optional).
// One workgroup per row, the updated row staged in LDS between the passes.
template <typename T>
__global__ void group_norm_pair_kernel(float* __restrict__ x, const T* __restrict__ a, const T* __restrict__ b,
                                       const float* __restrict__ w1, const float* __restrict__ w2,
                                       T* __restrict__ out1, T* __restrict__ out2, int W, int groups, float eps) {
  extern __shared__ float row[];          // [W] | per-group 1/rms [groups]
  __shared__ float scratch[16];
  float* rinv = row + W;
  const int64_t t = blockIdx.x;
  float* xr = x + t * W;
  const int gs = W / groups;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = xr[i];
    if (a != nullptr) v += ldf(a + t * W + i);
    if (b != nullptr) v += ldf(b + t * W + i);
    row[i] = v;
    if (a != nullptr) xr[i] = v;
  }
  __syncthreads();
  for (int g = 0; g < groups; ++g) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < gs; i += blockDim.x) { const float v = row[g * gs + i]; ss += v * v; }
    ss = block_sum(ss, scratch);
    if (threadIdx.x == 0) rinv[g] = 1.0f / sqrtf(ss / (float)gs + eps);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float n = row[i] * rinv[i / gs];
    stf(out1 + t * W + i, n * w1[i]);
    if (out2 != nullptr) stf(out2 + t * W + i, n * w2[i]);
  }
}

// 8-wide form (W and W/groups multiples of 8, 16-byte aligned rows): every
// thread keeps its chunks of the row in registers; the chunks' sums of squares
// go through LDS, one wave at a time adds up the chunks of a group in a fixed
// order, and each chunk is scaled by its group's factor. NC = chunks per thread.
template <typename T, int NC>
__global__ void group_norm_pair_v8_kernel(float* __restrict__ x, const T* __restrict__ a,
                                          const T* __restrict__ b, const float* __restrict__ w1,
                                          const float* __restrict__ w2, T* __restrict__ out1,
                                          T* __restrict__ out2, int W, int groups, float eps) {
  extern __shared__ float part[];         // [W/8] chunk sums | [groups] factors
  const int nchunk = W / 8, cpg = nchunk / groups;
  float* rinv = part + nchunk;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, nw = blockDim.x / WAVE;
  float v[NC][8];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int ch = threadIdx.x + c * blockDim.x;
    if (ch < nchunk) {
      ld8(x + t * W + ch * 8, v[c]);
      if (a != nullptr) {
        float u[8];
        ld8(a + t * W + ch * 8, u);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] += u[e];
        if (b != nullptr) {
          ld8(b + t * W + ch * 8, u);
#pragma unroll
          for (int e = 0; e < 8; ++e) v[c][e] += u[e];
        }
        st8(x + t * W + ch * 8, v[c]);
      }
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[c][e] * v[c][e];
      part[ch] = ss;
    }
  }
  __syncthreads();
  for (int g = wave; g < groups; g += nw) {
    float ss = 0.f;
    for (int i = lane; i < cpg; i += WAVE) ss += part[g * cpg + i];
    ss = wave_sum(ss);
    if (lane == 0) rinv[g] = 1.0f / sqrtf(ss / (float)(cpg * 8) + eps);
  }
  __syncthreads();
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    const int ch = threadIdx.x + c * blockDim.x;
    if (ch < nchunk) {
      const float r = rinv[ch / cpg];
      float ww[8], y[8];
      ld8(w1 + ch * 8, ww);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = v[c][e] * r * ww[e];
      st8(out1 + t * W + ch * 8, y);
      if (out2 != nullptr) {
        ld8(w2 + ch * 8, ww);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = v[c][e] * r * ww[e];
        st8(out2 + t * W + ch * 8, y);
      }
    }
  }
}

// ---- loop entry: x += a + b, out = [x | x0] in the activation type ---------------
template <typename T>
__global__ void cast_concat_kernel(T* __restrict__ out, float* __restrict__ x, const float* __restrict__ x0,
                                   const T* __restrict__ a, const T* __restrict__ b, int W) {
  const int64_t t = blockIdx.x;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float v = x[t * W + i];
    if (a != nullptr) {
      v += ldf(a + t * W + i);
      if (b != nullptr) v += ldf(b + t * W + i);
      x[t * W + i] = v;
    }
    stf(out + t * 2 * W + i, v);
    stf(out + t * 2 * W + W + i, x0[t * W + i]);
  }
}

// ---- per-head RMS norm, full-width weight, activated gate ------------------------
// o [T, H, S] fp32; out[t, h*S + i] = o / rms(o[t,h,:]) * w[h*S + i] * act(gate[t, h*S + i]);
// act = sigmoid (0) or silu (1). One wave per (row, head). With mt != nullptr the
// head rows of o are S + 1 wide: the last entry is a normaliser n.q and the
// head is first divided by max(|n.q|, e^-mt) + 1e-6 (the mlstm read-out).
template <typename T>
__global__ void head_rmsnorm_gate_kernel(T* __restrict__ out, const float* __restrict__ o,
                                         const float* __restrict__ w, const T* __restrict__ gate,
                                         const float* __restrict__ mt, int H, int S,
                                         int gate_stride, float eps, int gate_act) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + (t * H + h) * (mt != nullptr ? S + 1 : S);
  const float pre = mt != nullptr ? 1.0f / (fmaxf(fabsf(orow[S]), expf(-mt[t * H + h])) + 1e-6f) : 1.0f;
  float ss = 0.f;
  for (int i = lane; i < S; i += WAVE) { const float v = orow[i] * pre; ss += v * v; }
  ss = wave_sum(ss);
  const float r = pre / sqrtf(ss / (float)S + eps);
  const T* grow = gate + t * gate_stride + (int64_t)h * S;
  for (int i = lane; i < S; i += WAVE) {
    const float g = ldf(grow + i);
    const float ga = gate_act == 0 ? sigmoid_exact(g) : silu_exact(g);
    stf(out + (t * H + h) * S + i, orow[i] * r * w[(int64_t)h * S + i] * ga);
  }
}

// ---- token shift: mixes of a row with its predecessor -----------------------------
// out[s][t] = h[t] + (prev[t] - h[t]) * mu[s]; the first n_act mixes are written in
// the activation type, the rest in fp32. prev of a segment's first row is the
// carried row (zeros for a fresh sequence).
template <typename T>
__global__ void token_shift_mix_kernel(T* __restrict__ act, float* __restrict__ f32, const T* __restrict__ h,
                                       const float* __restrict__ mu, const T* __restrict__ shift_state,
                                       const int* __restrict__ slots, const int* __restrict__ cu,
                                       const int* __restrict__ seg_start, const int* __restrict__ token_seg,
                                       int T_, int W, int n, int n_act) {
  const int64_t t = blockIdx.x;
  const int b = token_seg[t];
  const bool first = t == cu[b];
  const bool fresh = seg_start[b] == 0;
  const T* prow = first ? shift_state + (int64_t)slots[b] * W : h + (t - 1) * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float hv = ldf(h + t * W + i);
    const float pv = (first && fresh) ? 0.f : ldf(prow + i);
    const float d = pv - hv;
    for (int s = 0; s < n; ++s) {
      const float v = hv + d * mu[(int64_t)s * W + i];
      if (s < n_act) stf(act + ((int64_t)s * T_ + t) * W + i, v);
      else f32[((int64_t)(s - n_act) * T_ + t) * W + i] = v;
    }
  }
}

// 8-wide form: one chunk of 8 columns per thread and iteration
template <typename T>
__global__ void token_shift_mix_v8_kernel(T* __restrict__ act, float* __restrict__ f32, const T* __restrict__ h,
                                          const float* __restrict__ mu, const T* __restrict__ shift_state,
                                          const int* __restrict__ slots, const int* __restrict__ cu,
                                          const int* __restrict__ seg_start, const int* __restrict__ token_seg,
                                          int T_, int W, int n, int n_act) {
  const int64_t t = blockIdx.x;
  const int b = token_seg[t];
  const bool first = t == cu[b];
  const bool fresh = seg_start[b] == 0;
  const T* prow = first ? shift_state + (int64_t)slots[b] * W : h + (t - 1) * W;
  for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
    float hv[8], d[8], m[8], y[8];
    ld8(h + t * W + i, hv);
    if (first && fresh) {
#pragma unroll
      for (int e = 0; e < 8; ++e) d[e] = -hv[e];
    } else {
      ld8(prow + i, d);
#pragma unroll
      for (int e = 0; e < 8; ++e) d[e] -= hv[e];
    }
    for (int s = 0; s < n; ++s) {
      ld8(mu + (int64_t)s * W + i, m);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = hv[e] + d[e] * m[e];
      if (s < n_act) st8(act + ((int64_t)s * T_ + t) * W + i, y);
      else st8(f32 + ((int64_t)(s - n_act) * T_ + t) * W + i, y);
    }
  }
}

template <typename T>
__global__ void shift_state_update_kernel(const T* __restrict__ h, T* __restrict__ shift_state,
                                          const int* __restrict__ slots, const int* __restrict__ cu, int W) {
  const int b = blockIdx.x;
  if (cu[b + 1] <= cu[b]) return;
  const T* src = h + (int64_t)(cu[b + 1] - 1) * W;
  T* dst = shift_state + (int64_t)slots[b] * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) dst[i] = src[i];
}

// ---- router --------------------------------------------------------------------
// One workgroup per row (the routing proper is its first wave's). s = softmax(z) over the N outputs; c = s + correction; the
// outputs form `gc` equal groups of neighbours, a group's score is its largest
// c, the best `gk` groups stay eligible; the `top` eligible outputs with the
// largest c are chosen (ties: the lower index). w = chosen s / (sum + 1e-20).
// The logits come from z [T, N], or (z == nullptr) are computed here in fp32
// as router [N, W] times the row of h. rowidx (optional) receives, for the
// all-experts form with E real experts over T_ rows, choice * T_ + row for a
// real expert and -1 for an identity expert.
#define ROUTE_MAX_N 256
template <typename T>
__global__ void __launch_bounds__(256) moe_route_kernel(int* __restrict__ idx, float* __restrict__ wout,
                                                        int* __restrict__ rowidx, const float* __restrict__ z,
                                                        const T* __restrict__ h,
                                                        const float* __restrict__ router,
                                                        const float* __restrict__ corr, int N, int W, int top,
                                                        int gc, int gk, int E, int T_, int vec,
                                                        int score_kind, int renorm) {
  __shared__ float cs[ROUTE_MAX_N], ss[ROUTE_MAX_N], gmax[ROUTE_MAX_N], zs[ROUTE_MAX_N];
  __shared__ int ok[ROUTE_MAX_N];
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, nw = blockDim.x / WAVE;
  // logits: every wave of the block takes outputs in turn; the routing proper is wave 0's
  if (z != nullptr) {
    for (int e = threadIdx.x; e < N; e += blockDim.x) zs[e] = z[t * N + e];
  } else {
    const T* hr = h + t * W;
    for (int e = wave; e < N; e += nw) {
      const float* rr = router + (int64_t)e * W;
      float acc = 0.f;
      if (vec) {
        for (int c = lane * 8; c < W; c += WAVE * 8) {
          float hv[8], rv[8];
          ld8(hr + c, hv);
          ld8(rr + c, rv);
#pragma unroll
          for (int k = 0; k < 8; ++k) acc += hv[k] * rv[k];
        }
      } else {
        for (int i = lane; i < W; i += WAVE) acc += ldf(hr + i) * rr[i];
      }
      acc = wave_sum(acc);
      if (lane == 0) zs[e] = acc;
    }
  }
  __syncthreads();
  const int per = N / gc;
  if (wave == 0 && score_kind == 0) {          // softmax over the outputs
    float mx = -INFINITY;
    for (int e = lane; e < N; e += WAVE) mx = fmaxf(mx, zs[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < N; e += WAVE) { const float p = expf(zs[e] - mx); ss[e] = p; sum += p; }
    sum = wave_sum(sum);
    for (int e = lane; e < N; e += WAVE) { ss[e] /= sum; cs[e] = ss[e] + (corr != nullptr ? corr[e] : 0.f); }
  } else if (wave == 0) {                      // sigmoid of each output
    for (int e = lane; e < N; e += WAVE) {
      ss[e] = sigmoid_exact(zs[e]);
      cs[e] = ss[e] + (corr != nullptr ? corr[e] : 0.f);
    }
  }
  __syncthreads();
  if (wave == 0) {
    for (int g = lane; g < gc; g += WAVE) {
      float m = -INFINITY;
      for (int i = 0; i < per; ++i) m = fmaxf(m, cs[g * per + i]);
      gmax[g] = m;
      ok[g] = 0;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int r = 0; r < gk; ++r) {
      int best = -1;
      for (int g = 0; g < gc; ++g)
        if (!ok[g] && (best < 0 || gmax[g] > gmax[best])) best = g;
      if (best >= 0) ok[best] = 1;
    }
  }
  __syncthreads();
  float wsum = 0.f, mine = 0.f;       // lane j of wave 0 keeps the j-th choice's score
  for (int r = 0; r < top; ++r) {
    if (wave == 0) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
      for (int e = lane; e < N; e += WAVE) {
        if (ok[e / per] && (cs[e] > bv)) { bv = cs[e]; bi = e; }     // ascending e: ties keep the lower index
      }
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) {
        const float ov = __shfl_xor(bv, off);
        const int oi = __shfl_xor(bi, off);
        if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
      }
      if (bi >= N) bi = 0;             // nothing comparable left (not-a-number scores): stay in range
      const float sv = ss[bi];
      wsum += sv;
      if (lane == r) mine = sv;
      if (lane == 0) {
        idx[t * top + r] = bi;
        if (rowidx != nullptr) rowidx[t * top + r] = bi < E ? bi * T_ + (int)t : -1;
        cs[bi] = -INFINITY;
      }
    }
    __syncthreads();
  }
  if (wave == 0 && lane < top) wout[t * top + lane] = renorm ? mine / (wsum + 1e-20f) : mine;
}

// ---- combine: out[t] = sum_j w[t,j] * (rowidx[t,j] >= 0 ? rows[rowidx[t,j]] : h[t]) ------
// w == nullptr: unweighted. extra != nullptr: + sigmoid(extra_gate[t]) * extra[t].
template <typename T>
__global__ void moe_combine_kernel(T* __restrict__ out, const T* __restrict__ rows, const T* __restrict__ h,
                                   const int* __restrict__ rowidx, const float* __restrict__ w,
                                   const T* __restrict__ extra, const T* __restrict__ extra_gate,
                                   int gate_stride, int W, int top) {
  const int64_t t = blockIdx.x;
  const float eg = extra != nullptr ? sigmoid_exact(ldf(extra_gate + t * gate_stride)) : 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < top; ++j) {
      const int r = rowidx[t * top + j];
      const float v = r >= 0 ? ldf(rows + (int64_t)r * W + i) : ldf(h + t * W + i);
      acc += w != nullptr ? w[t * top + j] * v : v;
    }
    if (extra != nullptr) acc += eg * ldf(extra + t * W + i);
    stf(out + t * W + i, acc);
  }
}

// the same combine with 8-wide accesses (W % 8 == 0, 16-byte aligned rows)
template <typename T>
__global__ void moe_combine_v8_kernel(T* __restrict__ out, const T* __restrict__ rows, const T* __restrict__ h,
                                      const int* __restrict__ rowidx, const float* __restrict__ w,
                                      const T* __restrict__ extra, const T* __restrict__ extra_gate,
                                      int gate_stride, int W, int top) {
  const int64_t t = blockIdx.x;
  const float eg = extra != nullptr ? sigmoid_exact(ldf(extra_gate + t * gate_stride)) : 0.f;
  for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, v[8];
    for (int j = 0; j < top; ++j) {
      const int r = rowidx[t * top + j];
      ld8(r >= 0 ? rows + (int64_t)r * W + i : h + t * W + i, v);
      const float wj = w != nullptr ? w[t * top + j] : 1.0f;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += w != nullptr ? wj * v[e] : v[e];
    }
    if (extra != nullptr) {
      ld8(extra + t * W + i, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += eg * v[e];
    }
    st8(out + t * W + i, acc);
  }
}

// ---- out[i] = h[src_row[i]] * scale[i]: expert inputs that carry their routing weight ------
template <typename T>
__global__ void scale_rows_kernel(T* __restrict__ out, const T* __restrict__ h, const int* __restrict__ src_row,
                                  const float* __restrict__ scale, int W) {
  const int64_t r = blockIdx.x;
  const T* src = h + (int64_t)src_row[r] * W;
  const float sc = scale[r];
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + r * W + i, ldf(src + i) * sc);
}

// ---- all-experts form of input-weighted experts: out[e, t] = w[t, j] * h[t] where expert e is
// row t's j-th choice, zero rows elsewhere. grid (E * T)
template <typename T>
__global__ void moe_spread_rows_kernel(T* __restrict__ out, const T* __restrict__ h, const int* __restrict__ idx,
                                       const float* __restrict__ w, int T_, int W, int top) {
  const int64_t r = blockIdx.x;
  const int e = (int)(r / T_), t = (int)(r - (int64_t)e * T_);
  float sc = 0.f;
  for (int j = 0; j < top; ++j)
    if (idx[t * top + j] == e) sc = w[t * top + j];
  const T* src = h + (int64_t)t * W;
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + r * W + i, sc != 0.f ? ldf(src + i) * sc : 0.f);
}

template <typename T>
__global__ void scale_rows_v8_kernel(T* __restrict__ out, const T* __restrict__ h,
                                     const int* __restrict__ src_row, const float* __restrict__ scale, int W) {
  const int64_t r = blockIdx.x;
  const T* src = h + (int64_t)src_row[r] * W;
  const float sc = scale[r];
  for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
    float v[8];
    ld8(src + i, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= sc;
    st8(out + r * W + i, v);
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

static inline int row_threads(int W) { return W >= 1024 ? 256 : (W >= 256 ? 128 : 64); }

extern "C" void seq_launch_embed_bigram(float* out, const int64_t* ids, const void* table, const void* bigram,
                                        float scale, int mul_prev, int mul_cur, int buckets, int* tok_state,
                                        const int* slots, const int* cu, const int* seg_start,
                                        const int* token_seg, int T_, int B, int W, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(embed_bigram_kernel<T>, dim3(T_), dim3(row_threads(W)), 0, st, out, ids,
                                        (const T*)table, (const T*)bigram, scale, mul_prev, mul_cur, buckets,
                                        tok_state, slots, cu, seg_start, token_seg, W);)
  if (bigram != nullptr)
    hipLaunchKernelGGL(tok_state_update_kernel, dim3((B + 63) / 64), dim3(64), 0, st, ids, tok_state, slots, cu, B);
}

extern "C" void seq_launch_group_norm_pair(float* x, const void* a, const void* b, const float* w1,
                                           const float* w2, void* out1, void* out2, int T_, int W, int groups,
                                           float eps, int is_f32, hipStream_t st) {
  const int nchunk = W / 8;
  if (W % 8 == 0 && (W / groups) % 8 == 0 && nchunk <= 2048 && aligned16(x) && aligned16(w1) &&
      aligned16(out1) && (a == nullptr || aligned16(a)) && (b == nullptr || aligned16(b)) &&
      (out2 == nullptr || (aligned16(out2) && aligned16(w2)))) {
    // one or two chunks per thread, whole waves
    int threads = nchunk <= 256 ? (nchunk + WAVE - 1) / WAVE * WAVE : ((nchunk + 1) / 2 + WAVE - 1) / WAVE * WAVE;
    const size_t lds8 = (size_t)(nchunk + groups) * sizeof(float);
    if (nchunk <= 256) {
      DISPATCH_T(is_f32, hipLaunchKernelGGL((group_norm_pair_v8_kernel<T, 1>), dim3(T_), dim3(threads), lds8, st,
                                            x, (const T*)a, (const T*)b, w1, w2, (T*)out1, (T*)out2, W, groups,
                                            eps);)
    } else {
      DISPATCH_T(is_f32, hipLaunchKernelGGL((group_norm_pair_v8_kernel<T, 2>), dim3(T_), dim3(threads), lds8, st,
                                            x, (const T*)a, (const T*)b, w1, w2, (T*)out1, (T*)out2, W, groups,
                                            eps);)
    }
    return;
  }
  const size_t lds = (size_t)(W + groups) * sizeof(float);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(group_norm_pair_kernel<T>, dim3(T_), dim3(row_threads(W)), lds, st, x,
                                        (const T*)a, (const T*)b, w1, w2, (T*)out1, (T*)out2, W, groups, eps);)
}

extern "C" void seq_launch_cast_concat(void* out, float* x, const float* x0, const void* a, const void* b,
                                       int T_, int W, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(cast_concat_kernel<T>, dim3(T_), dim3(row_threads(W)), 0, st, (T*)out, x,
                                        x0, (const T*)a, (const T*)b, W);)
}

extern "C" void seq_launch_head_rmsnorm_gate(void* out, const float* o, const float* w, const void* gate,
                                             const float* mt, int T_, int H, int S, int gate_stride, float eps,
                                             int gate_act, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(head_rmsnorm_gate_kernel<T>, dim3(T_, H), dim3(WAVE), 0, st, (T*)out, o,
                                        w, (const T*)gate, mt, H, S, gate_stride, eps, gate_act);)
}

extern "C" void seq_launch_token_shift_mix(void* act, float* f32, const void* h, const float* mu,
                                           void* shift_state, const int* slots, const int* cu,
                                           const int* seg_start, const int* token_seg, int T_, int B, int W,
                                           int n, int n_act, int is_f32, hipStream_t st) {
  const bool v8 = W % 8 == 0 && aligned16(h) && aligned16(mu) && aligned16(shift_state) &&
                  (act == nullptr || aligned16(act)) && (f32 == nullptr || aligned16(f32));
  const int th8 = W / 8 >= 256 ? 256 : ((W / 8 + WAVE - 1) / WAVE * WAVE);
  DISPATCH_T(is_f32,
             if (v8) hipLaunchKernelGGL(token_shift_mix_v8_kernel<T>, dim3(T_), dim3(th8), 0, st, (T*)act, f32,
                                        (const T*)h, mu, (const T*)shift_state, slots, cu, seg_start, token_seg, T_,
                                        W, n, n_act);
             else hipLaunchKernelGGL(token_shift_mix_kernel<T>, dim3(T_), dim3(row_threads(W)), 0, st, (T*)act, f32,
                                (const T*)h, mu, (const T*)shift_state, slots, cu, seg_start, token_seg, T_, W, n,
                                n_act);
             hipLaunchKernelGGL(shift_state_update_kernel<T>, dim3(B), dim3(row_threads(W)), 0, st, (const T*)h,
                                (T*)shift_state, slots, cu, W);)
}

extern "C" void seq_launch_moe_route(int* idx, float* w, int* rowidx, const float* z, const void* h,
                                     const float* router, const float* corr, int T_, int N, int W, int top,
                                     int gc, int gk, int E, int score_kind, int renorm, int is_f32,
                                     hipStream_t st) {
  const int vec = (h != nullptr && W % 8 == 0 && aligned16(h) && aligned16(router)) ? 1 : 0;
  const int threads = h != nullptr ? 256 : WAVE;
  DISPATCH_T(is_f32, hipLaunchKernelGGL(moe_route_kernel<T>, dim3(T_), dim3(threads), 0, st, idx, w, rowidx, z,
                                        (const T*)h, router, corr, N, W, top, gc, gk, E, T_, vec, score_kind,
                                        renorm);)
}

extern "C" void seq_launch_moe_combine(void* out, const void* rows, const void* h, const int* rowidx,
                                       const float* w, const void* extra, const void* extra_gate,
                                       int gate_stride, int T_, int W, int top, int is_f32, hipStream_t st) {
  if (W % 8 == 0 && aligned16(out) && aligned16(rows) && aligned16(h) && (extra == nullptr || aligned16(extra))) {
    const int threads = W / 8 >= 256 ? 256 : (W / 8 > 64 ? 128 : 64);
    DISPATCH_T(is_f32, hipLaunchKernelGGL(moe_combine_v8_kernel<T>, dim3(T_), dim3(threads), 0, st, (T*)out,
                                          (const T*)rows, (const T*)h, rowidx, w, (const T*)extra,
                                          (const T*)extra_gate, gate_stride, W, top);)
    return;
  }
  DISPATCH_T(is_f32, hipLaunchKernelGGL(moe_combine_kernel<T>, dim3(T_), dim3(row_threads(W)), 0, st, (T*)out,
                                        (const T*)rows, (const T*)h, rowidx, w, (const T*)extra,
                                        (const T*)extra_gate, gate_stride, W, top);)
}

extern "C" void seq_launch_moe_spread_rows(void* out, const void* h, const int* idx, const float* w, int E,
                                           int T_, int W, int top, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(moe_spread_rows_kernel<T>, dim3(E * T_), dim3(row_threads(W)), 0, st,
                                        (T*)out, (const T*)h, idx, w, T_, W, top);)
}

extern "C" void seq_launch_scale_rows(void* out, const void* h, const int* src_row, const float* scale, int n,
                                      int W, int is_f32, hipStream_t st) {
  if (W % 8 == 0 && aligned16(out) && aligned16(h)) {
    const int threads = W / 8 >= 256 ? 256 : (W / 8 > 64 ? 128 : 64);
    DISPATCH_T(is_f32, hipLaunchKernelGGL(scale_rows_v8_kernel<T>, dim3(n), dim3(threads), 0, st, (T*)out,
                                          (const T*)h, src_row, scale, W);)
    return;
  }
  DISPATCH_T(is_f32, hipLaunchKernelGGL(scale_rows_kernel<T>, dim3(n), dim3(row_threads(W)), 0, st, (T*)out,
                                        (const T*)h, src_row, scale, W);)
}
