// fp32-residual normalisation kernels and the clamped GLU activation.
// One workgroup per token row; rows are re-read from L1/L2 between passes
// instead of being held in registers, so any width works.

#include "seq_common.h"

// out[t] = rmsnorm(table[ids[t]] (+ pos_table[positions[t]])) * w   (fp32 residual stream)
template <typename T>
__global__ void embed_rmsnorm_kernel(float* __restrict__ out, const int64_t* __restrict__ ids,
                                     const T* __restrict__ table, const float* __restrict__ w,
                                     const T* __restrict__ pos_table, const int64_t* __restrict__ positions,
                                     int W, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = table + (int64_t)ids[t] * W;
  const T* prow = pos_table != nullptr ? pos_table + positions[t] * W : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float v = ldf(row + i) + (prow != nullptr ? ldf(prow + i) : 0.f);
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    out[(int64_t)t * W + i] = (ldf(row + i) + (prow != nullptr ? ldf(prow + i) : 0.f)) * r * w[i];
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
//   out = x                                  (w_next == nullptr, out != nullptr: the
//                                             stream itself in the activation type)
// y is staged in dynamic LDS (W floats).
template <typename T, bool DUAL>
__global__ void sandwich_residual_kernel(float* __restrict__ x, const T* __restrict__ a,
                                         const T* __restrict__ b, const float* __restrict__ wa,
                                         const float* __restrict__ wb, const float* __restrict__ w_post,
                                         const float* __restrict__ w_next, T* __restrict__ out,
                                         int W, float eps) {
  extern __shared__ __align__(16) float ybuf[];
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
  if (out == nullptr) return;
  if (w_next == nullptr) {
    for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + base + i, ybuf[i]);
    return;
  }
  ssx = block_sum(ssx, scratch);
  const float rx = 1.0f / sqrtf(ssx * invW + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + base + i, ybuf[i] * rx * w_next[i]);
}

// The same epilogue with 8-wide accesses (W % 8 == 0, 16-byte aligned rows).
template <typename T, bool DUAL>
__global__ void sandwich_residual_v8_kernel(float* __restrict__ x, const T* __restrict__ a,
                                            const T* __restrict__ b, const float* __restrict__ wa,
                                            const float* __restrict__ wb, const float* __restrict__ w_post,
                                            const float* __restrict__ w_next, T* __restrict__ out,
                                            int W, float eps) {
  extern __shared__ __align__(16) float ybuf[];
  __shared__ float scratch[16];
  const int64_t base = (int64_t)blockIdx.x * W;
  const float invW = 1.0f / (float)W;
  float ssy = 0.f;
  float va[8], vb[8], w1[8], w2[8], y[8];
  if (DUAL) {
    float sa = 0.f, sb = 0.f;
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
      ld8(a + base + i, va); ld8(b + base + i, vb);
#pragma unroll
      for (int e = 0; e < 8; ++e) { sa += va[e] * va[e]; sb += vb[e] * vb[e]; }
    }
    sa = block_sum(sa, scratch);
    sb = block_sum(sb, scratch);
    const float ra = 1.0f / sqrtf(sa * invW + eps), rb = 1.0f / sqrtf(sb * invW + eps);
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
      ld8(a + base + i, va); ld8(b + base + i, vb); ld8(wa + i, w1); ld8(wb + i, w2);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        y[e] = 0.5f * (va[e] * ra * w1[e] + vb[e] * rb * w2[e]);
        ssy += y[e] * y[e];
      }
      st8(ybuf + i, y);
    }
  } else {
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
      ld8(a + base + i, y);
#pragma unroll
      for (int e = 0; e < 8; ++e) ssy += y[e] * y[e];
      st8(ybuf + i, y);
    }
  }
  ssy = block_sum(ssy, scratch);
  const float ry = 1.0f / sqrtf(ssy * invW + eps);
  float ssx = 0.f;
  for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {   // each thread re-reads its own ybuf entries
    ld8(ybuf + i, y); ld8(x + base + i, va); ld8(w_post + i, w1);
#pragma unroll
    for (int e = 0; e < 8; ++e) { va[e] += y[e] * ry * w1[e]; ssx += va[e] * va[e]; }
    st8(x + base + i, va);
    st8(ybuf + i, va);
  }
  if (out == nullptr) return;
  if (w_next == nullptr) {
    for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) { ld8(ybuf + i, va); st8(out + base + i, va); }
    return;
  }
  ssx = block_sum(ssx, scratch);
  const float rx = 1.0f / sqrtf(ssx * invW + eps);
  for (int i = threadIdx.x * 8; i < W; i += blockDim.x * 8) {
    ld8(ybuf + i, va); ld8(w_next + i, w1);
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = va[e] * rx * w1[e];
    st8(out + base + i, y);
  }
}

// out[t, g*S + i] = o[t,g,i] / rms(o[t,g,:]) * w[i] * sigmoid(gate[t, g*S + i])
// gate_first: the gate is silu and comes before the norm, the weight spans the
// whole row: y = o * silu(gate); out = y / rms(y[t,g,:]) * w[g*S + i]
template <typename T>
__global__ void gated_rmsnorm_kernel(T* __restrict__ out, const float* __restrict__ o,
                                     const float* __restrict__ w, const T* __restrict__ gate,
                                     int S, int gate_stride, float eps, int gate_first) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, g = blockIdx.y, G = gridDim.y;
  const float* row = o + ((int64_t)t * G + g) * S;
  const T* grow = gate + (int64_t)t * gate_stride + (int64_t)g * S;
  float ss = 0.f;
  for (int i = threadIdx.x; i < S; i += blockDim.x) {
    float v = row[i];
    if (gate_first) v *= silu_exact(ldf(grow + i));
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)S + eps);
  T* orow = out + ((int64_t)t * G + g) * S;
  for (int i = threadIdx.x; i < S; i += blockDim.x) {
    const float gv = ldf(grow + i);
    stf(orow + i, gate_first ? row[i] * silu_exact(gv) * r * w[(int64_t)g * S + i]
                             : row[i] * r * w[i] * sigmoid_exact(gv));
  }
}

// 8-wide, single pass: each thread keeps its (up to two) chunks of the row in
// registers between the sum of squares and the scaling. One workgroup per row.
template <typename T>
__global__ void gated_rmsnorm_v8_kernel(T* __restrict__ out, const float* __restrict__ o,
                                        const float* __restrict__ w, const T* __restrict__ gate,
                                        int S, int gate_stride, float eps, int gate_first) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, g = blockIdx.y, G = gridDim.y;
  const float* row = o + ((int64_t)t * G + g) * S;
  const T* grow = gate + (int64_t)t * gate_stride + (int64_t)g * S;
  float v[2][8], ww[8], gg[8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int i = (threadIdx.x + c * blockDim.x) * 8;
    if (i < S) {
      ld8(row + i, v[c]);
      if (gate_first) {
        ld8(grow + i, gg);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] *= silu_exact(gg[e]);
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss += v[c][e] * v[c][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)S + eps);
  T* orow = out + ((int64_t)t * G + g) * S;
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const int i = (threadIdx.x + c * blockDim.x) * 8;
    if (i < S) {
      if (gate_first) {
        ld8(w + (int64_t)g * S + i, ww);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] = v[c][e] * r * ww[e];
      } else {
        ld8(w + i, ww); ld8(grow + i, gg);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] = v[c][e] * r * ww[e] * sigmoid_exact(gg[e]);
      }
      st8(orow + i, v[c]);
    }
  }
}

// Short rows (S = 8 * LPG, LPG a power of two <= 64): LPG lanes per row, 64/LPG
// rows per wave, reduction inside the lane group.
template <typename T>
__global__ void gated_rmsnorm_rows_kernel(T* __restrict__ out, const float* __restrict__ o,
                                          const float* __restrict__ w, const T* __restrict__ gate,
                                          int64_t rows, int G, int S, int LPG, int gate_stride, float eps,
                                          int gate_first) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t row = tid / LPG;
  const int i = (int)(tid - row * LPG) * 8;
  const bool on = row < rows;
  const int64_t t = row / G;
  const int g = (int)(row - t * G);
  float v[8], ww[8], gg[8];
  float ss = 0.f;
  if (on) {
    ld8(o + row * S + i, v);
    ld8(gate + t * gate_stride + (int64_t)g * S + i, gg);
    if (gate_first) {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] *= silu_exact(gg[e]);
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
  }
  for (int off = 1; off < LPG; off <<= 1) ss += __shfl_xor(ss, off);
  if (!on) return;
  const float r = 1.0f / sqrtf(ss / (float)S + eps);
  ld8(w + (gate_first ? (int64_t)g * S : 0) + i, ww);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = v[e] * r * ww[e] * (gate_first ? 1.0f : sigmoid_exact(gg[e]));
  st8(out + row * S + i, v);
}

// y = min(g, lim) * sigmoid(alpha * min(g, lim)) * (clamp(u, -lim, lim) + up_bias);
// lim = inf, alpha = 1, up_bias = 0 is silu(g) * u
template <typename T>
__global__ void clamped_glu_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                   const T* __restrict__ up, int64_t n, int cols, int stride,
                                   float limit, float alpha, float up_bias) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cols, c = i - r * cols;
    float g = fminf(ldf(gate + r * stride + c), limit);
    float u = fminf(fmaxf(ldf(up + r * stride + c), -limit), limit);
    stf(out + i, g * sigmoid_exact(alpha * g) * (u + up_bias));
  }
}

template <typename T>
__global__ void clamped_glu_v8_kernel(T* __restrict__ out, const T* __restrict__ gate,
                                      const T* __restrict__ up, int64_t n8, int cols8, int stride,
                                      float limit, float alpha, float up_bias) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cols8, c = (i - r * cols8) * 8;
    float g[8], u[8];
    ld8(gate + r * stride + c, g);
    ld8(up + r * stride + c, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gc = fminf(g[e], limit), uc = fminf(fmaxf(u[e], -limit), limit);
      g[e] = gc * sigmoid_exact(alpha * gc) * (uc + up_bias);
    }
    st8(out + i * 8, g);
  }
}

// tanh-form gelu: 0.5 z (1 + tanh(sqrt(2/pi) (z + 0.044715 z^3)))
__device__ __forceinline__ float gelu_tanh_exact(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}

template <typename T>
__global__ void gelu_tanh_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t n, int cols, int stride) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cols, c = i - r * cols;
    stf(out + i, gelu_tanh_exact(ldf(x + r * stride + c)));
  }
}

template <typename T>
__global__ void gelu_tanh_v8_kernel(T* __restrict__ out, const T* __restrict__ x, int64_t n8, int cols8,
                                    int stride) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t r = i / cols8, c = (i - r * cols8) * 8;
    float v[8];
    ld8(x + r * stride + c, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = gelu_tanh_exact(v[e]);
    st8(out + i * 8, v);
  }
}

// z <- z * scale, then cap * tanh(z / cap) when cap > 0 (fp32 logits, in place)
__global__ void scale_softcap_kernel(float* __restrict__ z, int64_t n, float scale, float cap) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const float v = z[i] * scale;
    z[i] = cap > 0.f ? cap * tanhf(v / cap) : v;
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

extern "C" void seq_launch_embed_rmsnorm(float* out, const int64_t* ids, const void* table,
                                         const float* w, const void* pos_table, const int64_t* positions,
                                         int T_, int W, float eps, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(embed_rmsnorm_kernel<T>, dim3(T_), dim3(256), 0, st, out, ids,
                                        (const T*)table, w, (const T*)pos_table, positions, W, eps);)
}

extern "C" void seq_launch_gelu_tanh(void* out, const void* x, int64_t rows, int cols, int stride, int is_f32,
                                     hipStream_t st) {
  if (cols % 8 == 0 && stride % 8 == 0 && aligned16(out) && aligned16(x)) {
    const int64_t n8 = rows * cols / 8;
    const int g8 = (int)((n8 + 255) / 256 < 16384 ? (n8 + 255) / 256 : 16384);
    DISPATCH_T(is_f32, hipLaunchKernelGGL(gelu_tanh_v8_kernel<T>, dim3(g8), dim3(256), 0, st, (T*)out,
                                          (const T*)x, n8, cols / 8, stride);)
    return;
  }
  const int64_t n = rows * cols;
  const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(gelu_tanh_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)out, (const T*)x,
                                        n, cols, stride);)
}

extern "C" void seq_launch_scale_softcap(float* z, int64_t n, float scale, float cap, hipStream_t st) {
  const int grid = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  hipLaunchKernelGGL(scale_softcap_kernel, dim3(grid), dim3(256), 0, st, z, n, scale, cap);
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
  const bool v8 = W % 8 == 0 && aligned16(x) && aligned16(a) && aligned16(b) && aligned16(out) &&
                  aligned16(wa) && aligned16(wb) && aligned16(w_post) && aligned16(w_next);
  if (v8 && b != nullptr) {
    DISPATCH_T(is_f32, hipLaunchKernelGGL((sandwich_residual_v8_kernel<T, true>), dim3(T_), dim3(256), lds, st,
                                          x, (const T*)a, (const T*)b, wa, wb, w_post, w_next, (T*)out, W, eps);)
  } else if (v8) {
    DISPATCH_T(is_f32, hipLaunchKernelGGL((sandwich_residual_v8_kernel<T, false>), dim3(T_), dim3(256), lds, st,
                                          x, (const T*)a, (const T*)b, wa, wb, w_post, w_next, (T*)out, W, eps);)
  } else if (b != nullptr) {
    DISPATCH_T(is_f32, hipLaunchKernelGGL((sandwich_residual_kernel<T, true>), dim3(T_), dim3(256), lds, st,
                                          x, (const T*)a, (const T*)b, wa, wb, w_post, w_next, (T*)out, W, eps);)
  } else {
    DISPATCH_T(is_f32, hipLaunchKernelGGL((sandwich_residual_kernel<T, false>), dim3(T_), dim3(256), lds, st,
                                          x, (const T*)a, (const T*)b, wa, wb, w_post, w_next, (T*)out, W, eps);)
  }
}

extern "C" void seq_launch_gated_rmsnorm(void* out, const float* o, const float* w, const void* gate,
                                         int T_, int G, int S, int gate_stride, float eps, int gate_first,
                                         int is_f32, hipStream_t st) {
  if (S % 8 == 0 && gate_stride % 8 == 0 && aligned16(out) && aligned16(o) && aligned16(w) && aligned16(gate)) {
    const int lpg = S / 8;
    if (lpg <= 64 && (lpg & (lpg - 1)) == 0) {
      const int64_t rows = (int64_t)T_ * G;
      const int grid = (int)((rows * lpg + 255) / 256);
      DISPATCH_T(is_f32, hipLaunchKernelGGL(gated_rmsnorm_rows_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)out,
                                            o, w, (const T*)gate, rows, G, S, lpg, gate_stride, eps, gate_first);)
      return;
    }
    int threads = ((lpg + 1) / 2 + WAVE - 1) / WAVE * WAVE;       // two chunks of 8 per thread
    if (threads <= 1024) {
      if (threads < WAVE) threads = WAVE;
      DISPATCH_T(is_f32, hipLaunchKernelGGL(gated_rmsnorm_v8_kernel<T>, dim3(T_, G), dim3(threads), 0, st,
                                            (T*)out, o, w, (const T*)gate, S, gate_stride, eps, gate_first);)
      return;
    }
  }
  const int threads = S >= 256 ? 256 : (S > 64 ? 128 : 64);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(gated_rmsnorm_kernel<T>, dim3(T_, G), dim3(threads), 0, st, (T*)out,
                                        o, w, (const T*)gate, S, gate_stride, eps, gate_first);)
}

extern "C" void seq_launch_gated_act(void* out, const void* gate, const void* up, int64_t rows, int cols,
                                     int stride, float limit, float alpha, float up_bias, int is_f32,
                                     hipStream_t st) {
  if (cols % 8 == 0 && stride % 8 == 0 && aligned16(out) && aligned16(gate) && aligned16(up)) {
    const int64_t n8 = rows * cols / 8;
    const int g8 = (int)((n8 + 255) / 256 < 16384 ? (n8 + 255) / 256 : 16384);
    DISPATCH_T(is_f32, hipLaunchKernelGGL(clamped_glu_v8_kernel<T>, dim3(g8), dim3(256), 0, st, (T*)out,
                                          (const T*)gate, (const T*)up, n8, cols / 8, stride, limit, alpha, up_bias);)
    return;
  }
  const int64_t n = rows * cols;
  const int grid = (int)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(clamped_glu_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)out,
                                        (const T*)gate, (const T*)up, n, cols, stride, limit, alpha, up_bias);)
}
