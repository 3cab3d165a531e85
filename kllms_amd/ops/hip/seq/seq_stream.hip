// Layer-normed sublayers over an fp32 stream with a short causal convolution on
// every sublayer's input and a depth-weighted sum of the layer results:
//
//   ln_residual_mix   y = x_in + ln(a) w_post  (post-norm + residual add), optionally
//                     kept as stream n and replaced by sum_j dwa[j] stream_j, and the
//                     (mean, rstd) of every resulting row for the norm that reads it next
//   ln_canon          h = (x - mean) rstd w  from those statistics, plus
//                     sum_j c[j] h_{t-K+1+j} over the row's predecessors (this step's
//                     rows, or the sequence's carried rows), cast to the GEMM type
//
// ln(v) = (v - mean) / sqrt(mean((v - mean)^2) + eps). The statistics travel
// between the two kernels so that the convolution, which needs the normed
// values of K rows, stays elementwise.

#include "seq_common.h"

template <int VEC, typename P>
__device__ __forceinline__ void ldv(const P* p, float v[VEC]) {
  if constexpr (VEC == 8) ld8(p, v);
  else v[0] = ldf(p);
}
template <int VEC, typename P>
__device__ __forceinline__ void stv(P* p, const float v[VEC]) {
  if constexpr (VEC == 8) st8(p, v);
  else stf(p, v[0]);
}

// grid T rows, dynamic LDS W floats (the row). a == nullptr: y = x_in.
// streams != nullptr: [n_prev + 1 or more, T, W]; stream n_prev takes y.
template <typename T, int VEC>
__global__ void ln_residual_mix_kernel(float* __restrict__ x_out, const float* __restrict__ x_in,
                                       const T* __restrict__ a, const float* __restrict__ w_post,
                                       float* __restrict__ stats, float* __restrict__ streams,
                                       const float* __restrict__ dwa, int n_prev, int64_t stream_stride,
                                       int W, float eps) {
  extern __shared__ __align__(16) float row[];
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * W;
  const float invW = 1.0f / (float)W;
  float v[VEC], u[VEC], w8[VEC];
  float mean_a = 0.f, r_a = 0.f;
  if (a != nullptr) {
    float s = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
      ldv<VEC>(a + base + i, v);
#pragma unroll
      for (int e = 0; e < VEC; ++e) { row[i + e] = v[e]; s += v[e]; }
    }
    mean_a = block_sum(s, scratch) * invW;
    float q = 0.f;
    for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
#pragma unroll
      for (int e = 0; e < VEC; ++e) { const float d = row[i + e] - mean_a; q += d * d; }
    }
    r_a = 1.0f / sqrtf(block_sum(q, scratch) * invW + eps);
  }
  float s = 0.f;
  for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
    ldv<VEC>(x_in + base + i, v);
    if (a != nullptr) {
      ldv<VEC>(w_post + i, w8);
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] += (row[i + e] - mean_a) * r_a * w8[e];
    }
    if (streams != nullptr) {
      stv<VEC>(streams + (int64_t)n_prev * stream_stride + base + i, v);
      float acc[VEC];
#pragma unroll
      for (int e = 0; e < VEC; ++e) acc[e] = 0.f;
      for (int j = 0; j < n_prev; ++j) {
        const float dj = dwa[j];
        ldv<VEC>(streams + (int64_t)j * stream_stride + base + i, u);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += dj * u[e];
      }
      const float dn = dwa[n_prev];
#pragma unroll
      for (int e = 0; e < VEC; ++e) v[e] = acc[e] + dn * v[e];
    }
    stv<VEC>(x_out + base + i, v);
#pragma unroll
    for (int e = 0; e < VEC; ++e) { row[i + e] = v[e]; s += v[e]; }
  }
  const float mean = block_sum(s, scratch) * invW;
  float q = 0.f;
  for (int i = threadIdx.x * VEC; i < W; i += blockDim.x * VEC) {
#pragma unroll
    for (int e = 0; e < VEC; ++e) { const float d = row[i + e] - mean; q += d * d; }
  }
  q = block_sum(q, scratch);
  if (threadIdx.x == 0) {
    stats[2 * (int64_t)blockIdx.x] = mean;
    stats[2 * (int64_t)blockIdx.x + 1] = 1.0f / sqrtf(q * invW + eps);
  }
}

// One thread per (row, VEC channels), grid-stride. K == 0: the norm alone.
// cw: taps-major [K, W], last row = the current token. hist: [slot][K-1][W]
// fp32 with hist_stride floats between slots, oldest row first.
template <typename T, int VEC>
__global__ void ln_canon_kernel(T* __restrict__ out, const float* __restrict__ x, const float* __restrict__ stats,
                                const float* __restrict__ w, const float* __restrict__ cw,
                                const float* __restrict__ hist, int64_t hist_stride,
                                const int* __restrict__ slots, const int* __restrict__ cu,
                                const int* __restrict__ seg_start, const int* __restrict__ token_seg,
                                int64_t n, int W, int K) {
  const int WV = W / VEC;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < n;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int t = (int)(idx / WV), c = (int)(idx - (int64_t)t * WV) * VEC;
    float xv[VEC], wv[VEC], acc[VEC], hv[VEC], cv[VEC], cur[VEC];
    ldv<VEC>(w + c, wv);
    ldv<VEC>(x + (int64_t)t * W + c, xv);
    const float m = stats[2 * (int64_t)t], r = stats[2 * (int64_t)t + 1];
#pragma unroll
    for (int e = 0; e < VEC; ++e) { cur[e] = (xv[e] - m) * r * wv[e]; acc[e] = cur[e]; }
    if (K > 0) {
      const int b = token_seg[t];
      const int i = t - cu[b];
      const bool fresh = seg_start[b] == 0;
      const float* hs = hist + (int64_t)slots[b] * hist_stride;
      for (int j = 0; j < K; ++j) {
        const int back = K - 1 - j;
        if (back > 0) {
          if (i - back >= 0) {
            const int64_t tt = t - back;
            ldv<VEC>(x + tt * W + c, xv);
            const float m2 = stats[2 * tt], r2 = stats[2 * tt + 1];
#pragma unroll
            for (int e = 0; e < VEC; ++e) hv[e] = (xv[e] - m2) * r2 * wv[e];
          } else if (!fresh) {
            ldv<VEC>(hs + (int64_t)(K - 1 + (i - back)) * W + c, hv);
          } else {
            continue;
          }
        } else {
#pragma unroll
          for (int e = 0; e < VEC; ++e) hv[e] = cur[e];
        }
        ldv<VEC>(cw + (int64_t)j * W + c, cv);
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[e] += cv[e] * hv[e];
      }
    }
    stv<VEC>(out + (int64_t)t * W + c, acc);
  }
}

// new history = last K-1 normed rows of (old history ++ this segment's rows);
// one thread per (segment, channel) reads everything it needs before it writes.
#define CANON_MAX_TAPS 16
__global__ void canon_state_update_kernel(const float* __restrict__ x, const float* __restrict__ stats,
                                          const float* __restrict__ w, float* __restrict__ hist,
                                          int64_t hist_stride, const int* __restrict__ slots,
                                          const int* __restrict__ cu, const int* __restrict__ seg_start, int B,
                                          int W, int K) {
  const int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (int64_t)B * W) return;
  const int b = (int)(idx / W), c = (int)(idx - (int64_t)b * W);
  const int t0 = cu[b], L = cu[b + 1] - t0;
  if (L == 0) return;
  const bool fresh = seg_start[b] == 0;
  float* hs = hist + (int64_t)slots[b] * hist_stride;
  float tmp[CANON_MAX_TAPS];
  for (int j = 0; j < K - 1; ++j) {
    const int src = L - (K - 1) + j;
    if (src >= 0) {
      const int64_t t = t0 + src;
      tmp[j] = (x[t * W + c] - stats[2 * t]) * stats[2 * t + 1] * w[c];
    } else {
      tmp[j] = fresh ? 0.f : hs[(int64_t)(K - 1 + src) * W + c];
    }
  }
  for (int j = 0; j < K - 1; ++j) hs[(int64_t)j * W + c] = tmp[j];
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

extern "C" void seq_launch_ln_residual_mix(float* x_out, const float* x_in, const void* a, const float* w_post,
                                           float* stats, float* streams, const float* dwa, int n_prev,
                                           int64_t stream_stride, int T_, int W, float eps, int is_f32,
                                           hipStream_t st) {
  const size_t lds = (size_t)W * sizeof(float);
  const bool v8 = W % 8 == 0 && aligned16(x_out) && aligned16(x_in) && (a == nullptr || aligned16(a)) &&
                  (w_post == nullptr || aligned16(w_post)) &&
                  (streams == nullptr || (aligned16(streams) && stream_stride % 4 == 0));
  if (v8) {
    const int threads = W / 8 >= 256 ? 256 : ((W / 8 + WAVE - 1) / WAVE * WAVE);
    DISPATCH_T(is_f32, hipLaunchKernelGGL((ln_residual_mix_kernel<T, 8>), dim3(T_), dim3(threads), lds, st, x_out,
                                          x_in, (const T*)a, w_post, stats, streams, dwa, n_prev, stream_stride, W,
                                          eps);)
  } else {
    const int threads = W >= 256 ? 256 : ((W + WAVE - 1) / WAVE * WAVE);
    DISPATCH_T(is_f32, hipLaunchKernelGGL((ln_residual_mix_kernel<T, 1>), dim3(T_), dim3(threads), lds, st, x_out,
                                          x_in, (const T*)a, w_post, stats, streams, dwa, n_prev, stream_stride, W,
                                          eps);)
  }
}

extern "C" void seq_launch_ln_canon(void* out, const float* x, const float* stats, const float* w,
                                    const float* cw, float* hist, int64_t hist_stride, const int* slots,
                                    const int* cu, const int* seg_start, const int* token_seg, int T_, int B,
                                    int W, int K, int is_f32, hipStream_t st) {
  const bool v8 = W % 8 == 0 && aligned16(out) && aligned16(x) && aligned16(w) &&
                  (K == 0 || (aligned16(cw) && (K == 1 || (aligned16(hist) && hist_stride % 4 == 0))));
  if (v8) {
    const int64_t n = (int64_t)T_ * (W / 8);
    const int grid = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    DISPATCH_T(is_f32, hipLaunchKernelGGL((ln_canon_kernel<T, 8>), dim3(grid), dim3(256), 0, st, (T*)out, x, stats,
                                          w, cw, hist, hist_stride, slots, cu, seg_start, token_seg, n, W, K);)
  } else {
    const int64_t n = (int64_t)T_ * W;
    const int grid = (int)((n + 255) / 256 < 16384 ? (n + 255) / 256 : 16384);
    DISPATCH_T(is_f32, hipLaunchKernelGGL((ln_canon_kernel<T, 1>), dim3(grid), dim3(256), 0, st, (T*)out, x, stats,
                                          w, cw, hist, hist_stride, slots, cu, seg_start, token_seg, n, W, K);)
  }
  if (K > 1) {
    const int grid2 = (int)(((int64_t)B * W + 255) / 256);
    hipLaunchKernelGGL(canon_state_update_kernel, dim3(grid2), dim3(256), 0, st, x, stats, w, hist, hist_stride,
                       slots, cu, seg_start, B, W, K);
  }
}
