// Rotary (interleaved pairs, partial width) + paged K/V store, q/k head norm +
// paged store, and masked softmax attention over the paged cache (block-local
// or sliding-window mask with kept first tokens, optional sink term). One kernel serves prompt portions,
// single decoded tokens and mixed batches: every query row finds its keys
// through its segment's block table, so the result does not depend on how the
// prompt was cut into steps.

#include "seq_common.h"

// grid (T, H + G), 64 threads. Heads 0..H-1 are query heads (rotated in place),
// H..H+G-1 key heads: rotated copy -> k_cache, value row (v, or the un-rotated
// key when v == nullptr) -> v_cache. angle = float(pos) * inv_freq[i], fp32.
template <typename T>
__global__ void rope_pairs_store_kernel(T* __restrict__ q, const T* __restrict__ k,
                                        const T* __restrict__ v, const int64_t* __restrict__ positions,
                                        const float* __restrict__ inv_freq, T* __restrict__ k_cache,
                                        T* __restrict__ v_cache, const int64_t* __restrict__ slots,
                                        T* __restrict__ kv_fresh, int H, int G, int D, int Dv, int R, int BS,
                                        int q_stride, int k_stride, int v_stride) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float pos = (float)positions[t];
  if (h < H) {
    T* row = q + (int64_t)t * q_stride + (int64_t)h * D;
    for (int i = threadIdx.x; i < R; i += blockDim.x) {
      float s, c;
      sincosf(pos * inv_freq[i], &s, &c);
      const float u = ldf(row + 2 * i), w = ldf(row + 2 * i + 1);
      stf(row + 2 * i, u * c - w * s);
      stf(row + 2 * i + 1, w * c + u * s);
    }
    return;
  }
  const int g = h - H;
  const int64_t slot = slots[t];
  const int64_t blk = slot / BS, off = slot % BS;
  const T* krow = k + (int64_t)t * k_stride + (int64_t)g * D;
  T* kc = k_cache + ((blk * G + g) * BS + off) * D;
  T* vc = v_cache + ((blk * G + g) * BS + off) * Dv;
  // optional packed copy of this step's rotated keys and values,
  // [T, 2, G, D] (needs Dv == D): the dense prefill kernel reads it
  T* fk = kv_fresh ? kv_fresh + (((int64_t)t * 2 + 0) * G + g) * D : nullptr;
  T* fv = kv_fresh ? kv_fresh + (((int64_t)t * 2 + 1) * G + g) * D : nullptr;
  const T* vrow = v != nullptr ? v + (int64_t)t * v_stride + (int64_t)g * Dv : krow;
  for (int i = threadIdx.x; i < Dv; i += blockDim.x) {
    vc[i] = vrow[i];
    if (fv) fv[i] = vrow[i];
  }
  for (int i = threadIdx.x; i < R; i += blockDim.x) {
    float s, c;
    sincosf(pos * inv_freq[i], &s, &c);
    const float u = ldf(krow + 2 * i), w = ldf(krow + 2 * i + 1);
    stf(kc + 2 * i, u * c - w * s);
    stf(kc + 2 * i + 1, w * c + u * s);
    if (fk) { fk[2 * i] = kc[2 * i]; fk[2 * i + 1] = kc[2 * i + 1]; }
  }
  for (int i = 2 * R + threadIdx.x; i < D; i += blockDim.x) {
    kc[i] = krow[i];
    if (fk) fk[i] = krow[i];
  }
}

// grid (T, H + G), one wave per (row, head): RMS norm over the head's D
// entries with a weight shared by the heads. Query heads are normed in place;
// key heads go normed into k_cache, their value rows into v_cache.
template <typename T>
__global__ void qk_norm_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                     const float* __restrict__ wq, const float* __restrict__ wk, float eps,
                                     T* __restrict__ k_cache, T* __restrict__ v_cache,
                                     const int64_t* __restrict__ slots, int H, int G, int D, int Dv, int BS,
                                     int q_stride, int k_stride, int v_stride) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool is_q = h < H;
  const int g = h - H;
  const T* src = is_q ? q + (int64_t)t * q_stride + (int64_t)h * D : k + (int64_t)t * k_stride + (int64_t)g * D;
  float ss = 0.f;
  for (int i = lane; i < D; i += WAVE) { const float x = ldf(src + i); ss += x * x; }
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)D + eps);
  if (is_q) {
    T* dst = q + (int64_t)t * q_stride + (int64_t)h * D;
    for (int i = lane; i < D; i += WAVE) stf(dst + i, ldf(src + i) * r * wq[i]);
    return;
  }
  const int64_t slot = slots[t];
  const int64_t blk = slot / BS, off = slot % BS;
  T* kc = k_cache + ((blk * G + g) * BS + off) * D;
  T* vc = v_cache + ((blk * G + g) * BS + off) * Dv;
  for (int i = lane; i < D; i += WAVE) stf(kc + i, ldf(src + i) * r * wk[i]);
  const T* vrow = v + (int64_t)t * v_stride + (int64_t)g * Dv;
  for (int i = lane; i < Dv; i += WAVE) vc[i] = vrow[i];
}

// The keys that position p sees, as nk kept first positions 0..nk-1 followed by
// lo..p. mask_kind 0: lo = the start of p's aligned block of mask_size
// positions, nothing kept. mask_kind 1: a window of mask_size positions ending
// at p, plus the first keep_first positions of the sequence. mask_size 0 =
// plain causal. Visible key number u (0 <= u < nk + p - lo + 1) is position
// u < nk ? u : lo + u - nk.
//
// mask_kind 2: a window of mask_size positions ending at p, and before it one
// pooled entry per aligned run of ``run`` positions that ends before the window
// (run u covers u*run .. u*run + run - 1; it is seen when its last position is
// <= p - mask_size). Visible key u < nk is then pooled run u, not a position.
__device__ __forceinline__ void mask_range(int mask_kind, int mask_size, int keep_first, int run, int p,
                                           int& lo, int& nk) {
  lo = 0; nk = 0;
  if (mask_size <= 0) return;
  if (mask_kind == 0) { lo = (p / mask_size) * mask_size; return; }
  lo = max(0, p - mask_size + 1);
  nk = mask_kind == 2 ? (run > 0 ? lo / run : 0) : min(keep_first, lo);
}

// Row of visible key u in the cache it lives in: >= 0 a token row of k_cache /
// v_cache, <= -2 row -(r + 2) of the pooled caches. A pooled run lives in the
// page of its last token, counted from the first run that ends in that page.
__device__ __forceinline__ int visible_row(int u, int nk, int lo, int mask_kind, int run, int PB,
                                           const int* __restrict__ bt, int G, int g, int BS) {
  if (u < nk && mask_kind == 2) {
    const int pg = ((u + 1) * run - 1) / BS;
    return -(((bt[pg] * G + g) * PB + (u - (pg * BS) / run)) + 2);
  }
  const int j = u < nk ? u : lo + (u - nk);
  return (bt[j / BS] * G + g) * BS + (j % BS);
}

__device__ __forceinline__ float softcapped(float s, float cap) { return cap > 0.f ? cap * tanhf(s / cap) : s; }

// grid (T, H), one wave per (query row, head). The visible keys in tiles of
// 64: lane u scores visible key tile*64 + u (q staged in LDS), the tile's weights
// go through LDS, then lanes own output dims and sweep the tile's value rows.
// Online softmax in fp32; with a sink the running (max, sum) starts at (0, 1):
// one more key of score 0 that carries no value. Optional sigmoid gate on the
// output: gate_kind 1 = one logit per head [T, H], 2 = per element [T, H*Dv].
#define ATTN_MAX_ACC 8   // Dv <= 512
template <typename T>
__global__ void attn_blocklocal_paged_kernel(T* __restrict__ out, const T* __restrict__ q,
                                             const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                             const int* __restrict__ block_tables,
                                             const int* __restrict__ token_seg,
                                             const int64_t* __restrict__ positions,
                                             const T* __restrict__ gate, const int* __restrict__ row_map,
                                             const float* __restrict__ pool_k, const float* __restrict__ pool_v,
                                             int run, int PB, float softcap,
                                             float scale, int mask_kind, int mask_size, int keep_first,
                                             int sink, int gate_kind,
                                             int H, int G, int D, int Dv, int BS, int bt_stride,
                                             int q_stride, int gate_stride) {
  extern __shared__ float lds[];       // q [D] | p [64] | key row index [64] (as int)
  float* qs = lds;
  float* ps = lds + D;
  int* rows = (int*)(ps + WAVE);
  // row_map (optional): the rows this launch serves; the others belong to
  // the dense prefill kernel
  const int t = row_map ? row_map[blockIdx.x] : blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const int g = h / (H / G);
  const int p = (int)positions[t];
  int lo, nk;
  mask_range(mask_kind, mask_size, keep_first, run, p, lo, nk);
  const int total = nk + (p - lo + 1);
  const int* bt = block_tables + (int64_t)token_seg[t] * bt_stride;
  const T* qrow = q + (int64_t)t * q_stride + (int64_t)h * D;
  for (int i = lane; i < D; i += WAVE) qs[i] = ldf(qrow + i) * scale;
  __syncthreads();

  float acc[ATTN_MAX_ACC];
#pragma unroll
  for (int i = 0; i < ATTN_MAX_ACC; ++i) acc[i] = 0.f;
  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  for (int base = 0; base < total; base += WAVE) {
    const int u = base + lane;
    float s = -INFINITY;
    int row = -1;
    if (u < total) {
      row = visible_row(u, nk, lo, mask_kind, run, PB, bt, G, g, BS);
      float d = 0.f;
      if (row >= 0) {
        const T* kr = k_cache + (int64_t)row * D;
        for (int i = 0; i < D; ++i) d += qs[i] * ldf(kr + i);
      } else {
        const float* kr = pool_k + (int64_t)(-(row + 2)) * D;
        for (int i = 0; i < D; ++i) d += qs[i] * kr[i];
      }
      s = softcapped(d, softcap);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float w = u < total ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);        // m = -inf on the first tile -> 0
    l = l * corr + wave_sum(w);
    m = m_new;
    ps[lane] = w;
    rows[lane] = row;
    __syncthreads();
    const int n = min(WAVE, total - base);
#pragma unroll
    for (int i = 0; i < ATTN_MAX_ACC; ++i) acc[i] *= corr;
    for (int jj = 0; jj < n; ++jj) {
      const float pw = ps[jj];
      const int rr = rows[jj];
      const T* vr = v_cache + (int64_t)(rr >= 0 ? rr : 0) * Dv;
      const float* vp = pool_v + (int64_t)(rr >= 0 ? 0 : -(rr + 2)) * Dv;
#pragma unroll
      for (int i = 0; i < ATTN_MAX_ACC; ++i) {
        const int d = lane + i * WAVE;
        if (d < Dv) acc[i] += pw * (rr >= 0 ? ldf(vr + d) : vp[d]);
      }
    }
    __syncthreads();
  }
  float gsc = 1.0f / l;
  if (gate_kind == 1) gsc *= sigmoid_exact(ldf(gate + (int64_t)t * gate_stride + h));
  T* orow = out + ((int64_t)t * H + h) * Dv;
  const T* grow = gate + (int64_t)t * gate_stride + (int64_t)h * Dv;
#pragma unroll
  for (int i = 0; i < ATTN_MAX_ACC; ++i) {
    const int d = lane + i * WAVE;
    if (d < Dv) stf(orow + d, acc[i] * gsc * (gate_kind == 2 ? sigmoid_exact(ldf(grow + d)) : 1.0f));
  }
}

// The same attention with coalesced 8-wide accesses — the decode kernel (and
// the one for continuing rows of a prompt portion). Needs D and Dv multiples
// of 8 with D/8 and Dv/8 powers of two <= 64, 16-byte aligned rows.
//   scores: LPK = D/8 lanes share one key (each holds 8 dims of q in registers
//           and loads 16 B of the key row), 64/LPK keys per pass, the partial
//           dots are summed inside the lane group;
//   values: LPV = Dv/8 lanes share one key's value row, 64/LPV keys per pass,
//           each lane accumulates 8 output dims; the key groups are summed
//           once at the end.
// Tiles of 64 keys, online softmax in fp32 as above; four waves per
// (row, head) share the tiles and merge at the end.
#define ATTN_V8_WAVES 4
template <typename T>
__global__ void __launch_bounds__(WAVE * ATTN_V8_WAVES) attn_blocklocal_paged_v8_kernel(
    T* __restrict__ out, const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, const int* __restrict__ token_seg,
    const int64_t* __restrict__ positions, const T* __restrict__ gate, const int* __restrict__ row_map,
    const float* __restrict__ pool_k, const float* __restrict__ pool_v, int run, int PB, float softcap,
    float* __restrict__ part_o, float* __restrict__ part_ml,
    float scale, int mask_kind, int mask_size, int keep_first, int sink, int gate_kind, int H, int G, int D,
    int Dv, int BS, int bt_stride, int q_stride, int gate_stride) {
  // gridDim.z > 1 (steps of few rows): the workgroups of one (row, head) take
  // contiguous shares of its key tiles and leave unnormalised partial results
  // (sums relative to the share's maximum, that maximum and the sum of weights)
  // in part_o [T, H, Z, Dv] / part_ml [T, H, Z, 2]; attn_split_merge_kernel
  // combines them in a fixed order.
  // The block's waves take the key tiles in turn (tile r*NW + wave in pass
  // r), each with its own running max / sum / accumulator; the partial
  // results are merged through LDS at the end. Every wave runs every pass —
  // a wave without a tile only keeps the barriers company.
  constexpr int NW = ATTN_V8_WAVES;
  __shared__ float ps_[NW][WAVE];
  __shared__ int rows_[NW][WAVE];
  __shared__ float part_m[NW], part_l[NW];
  __shared__ float part_acc[NW][512];
  const int t = row_map ? row_map[blockIdx.x] : blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  float* ps = ps_[wave];
  int* rows = rows_[wave];
  const int g = h / (H / G);
  const int p = (int)positions[t];
  int lo, nk;
  mask_range(mask_kind, mask_size, keep_first, run, p, lo, nk);
  const int total = nk + (p - lo + 1);
  const int* bt = block_tables + (int64_t)token_seg[t] * bt_stride;
  const int LPK = D / 8, KPI = WAVE / LPK, kpart = lane % LPK, kgrp = lane / LPK;
  const int LPV = Dv / 8, KPV = WAVE / LPV, vpart = lane % LPV, vgrp = lane / LPV;
  float qv[8];
  ld8(q + (int64_t)t * q_stride + (int64_t)h * D + kpart * 8, qv);
#pragma unroll
  for (int e = 0; e < 8; ++e) qv[e] *= scale;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  // the sink is one more key of score 0 without a value, held by wave 0
  const bool sunk = sink && wave == 0 && blockIdx.z == 0;
  float m = sunk ? 0.f : -INFINITY, l = sunk ? 1.f : 0.f;
  const int ntiles = (total + WAVE - 1) / WAVE;
  const int per_share = (ntiles + (int)gridDim.z - 1) / (int)gridDim.z;
  const int tile0 = (int)blockIdx.z * per_share, tile1 = min(ntiles, tile0 + per_share);
  for (int r = 0; tile0 + r * NW < tile1; ++r) {
    const int tile = tile0 + r * NW + wave;
    const int base = tile * WAVE;
    const int n = tile < tile1 ? min(WAVE, total - base) : 0;   // 0: no tile for this wave in this pass
    const int u = base + lane;
    rows[lane] = (n > 0 && u < total) ? visible_row(u, nk, lo, mask_kind, run, PB, bt, G, g, BS) : -1;
    __syncthreads();
    for (int it = 0; it * KPI < n; ++it) {
      const int key = it * KPI + kgrp;
      float d = 0.f;
      if (key < n) {
        float kv[8];
        const int rr = rows[key];
        if (rr >= 0) ld8(k_cache + (int64_t)rr * D + kpart * 8, kv);
        else ld8(pool_k + (int64_t)(-(rr + 2)) * D + kpart * 8, kv);
#pragma unroll
        for (int e = 0; e < 8; ++e) d += qv[e] * kv[e];
      }
      for (int off = 1; off < LPK; off <<= 1) d += __shfl_xor(d, off);
      if (kpart == 0 && key < n) ps[key] = softcapped(d, softcap);
    }
    __syncthreads();
    float w = 0.f, corr = 1.f;
    if (n > 0) {                                      // uniform over the wave
      const float s = lane < n ? ps[lane] : -INFINITY;
      const float m_new = fmaxf(m, wave_max(s));
      w = lane < n ? expf(s - m_new) : 0.f;
      corr = expf(m - m_new);                         // m = -inf on the wave's first tile -> 0
      l = l * corr + wave_sum(w);
      m = m_new;
    }
    __syncthreads();                                  // every lane has read its score
    ps[lane] = w;
    __syncthreads();
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= corr;
    for (int it = 0; it * KPV < n; ++it) {
      const int key = it * KPV + vgrp;
      if (key < n) {
        float vv[8];
        const int rr = rows[key];
        if (rr >= 0) ld8(v_cache + (int64_t)rr * Dv + vpart * 8, vv);
        else ld8(pool_v + (int64_t)(-(rr + 2)) * Dv + vpart * 8, vv);
        const float pw = ps[key];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += pw * vv[e];
      }
    }
    __syncthreads();
  }
  for (int off = LPV; off < WAVE; off <<= 1) {
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += __shfl_xor(acc[e], off);
  }
  // merge the waves' partial softmaxes
  if (lane == 0) { part_m[wave] = m; part_l[wave] = l; }
  if (vgrp == 0) {
#pragma unroll
    for (int e = 0; e < 8; ++e) part_acc[wave][vpart * 8 + e] = acc[e];
  }
  __syncthreads();
  if (wave == 0 && vgrp == 0) {
    float M = part_m[0];
#pragma unroll
    for (int w2 = 1; w2 < NW; ++w2) M = fmaxf(M, part_m[w2]);
    float L = 0.f, o8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w2 = 0; w2 < NW; ++w2) {
      const float f = part_l[w2] > 0.f ? expf(part_m[w2] - M) : 0.f;   // a wave that saw no key
      L += part_l[w2] * f;
#pragma unroll
      for (int e = 0; e < 8; ++e) o8[e] += part_acc[w2][vpart * 8 + e] * f;
    }
    if (gridDim.z > 1) {
      const int64_t pz = ((int64_t)t * H + h) * gridDim.z + blockIdx.z;
      if (vpart == 0) { part_ml[2 * pz] = M; part_ml[2 * pz + 1] = L; }
      st8(part_o + pz * Dv + vpart * 8, o8);
      return;
    }
    float gsc = 1.0f / L;
    if (gate_kind == 1) gsc *= sigmoid_exact(ldf(gate + (int64_t)t * gate_stride + h));
#pragma unroll
    for (int e = 0; e < 8; ++e) o8[e] *= gsc;
    if (gate_kind == 2) {
      float g8[8];
      ld8(gate + (int64_t)t * gate_stride + (int64_t)h * Dv + vpart * 8, g8);
#pragma unroll
      for (int e = 0; e < 8; ++e) o8[e] *= sigmoid_exact(g8[e]);
    }
    st8(out + ((int64_t)t * H + h) * Dv + vpart * 8, o8);
  }
}

// Merge of the key shares of one (row, head): grid (T, H), one thread per 8
// output dims. out = sum_z o_z e^(m_z - M) / sum_z l_z e^(m_z - M), M = max m_z,
// summed over z in order; a share that saw no key (l = 0) counts for nothing.
template <typename T>
__global__ void attn_split_merge_kernel(T* __restrict__ out, const float* __restrict__ part_o,
                                        const float* __restrict__ part_ml, int H, int Dv, int nsplit) {
  const int t = blockIdx.x, h = blockIdx.y;
  const int64_t base = ((int64_t)t * H + h) * nsplit;
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z) if (part_ml[2 * (base + z) + 1] > 0.f) M = fmaxf(M, part_ml[2 * (base + z)]);
  float L = 0.f;
  for (int z = 0; z < nsplit; ++z) {
    const float lz = part_ml[2 * (base + z) + 1];
    if (lz > 0.f) L += lz * expf(part_ml[2 * (base + z)] - M);
  }
  const float inv = 1.0f / L;
  for (int d = threadIdx.x * 8; d < Dv; d += blockDim.x * 8) {
    float o8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, v[8];
    for (int z = 0; z < nsplit; ++z) {
      const float lz = part_ml[2 * (base + z) + 1];
      if (lz > 0.f) {
        const float f = expf(part_ml[2 * (base + z)] - M);
        ld8(part_o + (base + z) * Dv + d, v);
#pragma unroll
        for (int e = 0; e < 8; ++e) o8[e] += v[e] * f;
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) o8[e] *= inv;
    st8(out + ((int64_t)t * H + h) * Dv + d, o8);
  }
}

// out[t, h, :] *= sigmoid(gate[t, h]) — the per-head output gate for rows
// whose attention came from a kernel without it
template <typename T>
__global__ void head_gate_kernel(T* __restrict__ out, const T* __restrict__ gate, int64_t n, int H, int Dv,
                                 int gate_stride) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / Dv;
    const int64_t t = th / H;
    const int h = (int)(th - t * H);
    stf(out + i, ldf(out + i) * sigmoid_exact(ldf(gate + t * gate_stride + h)));
  }
}

template <typename T>
__global__ void head_gate_v8_kernel(T* __restrict__ out, const T* __restrict__ gate, int64_t n8, int H, int Dv8,
                                    int gate_stride) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n8;
       i += (int64_t)gridDim.x * blockDim.x) {
    const int64_t th = i / Dv8;
    const int64_t t = th / H;
    const int h = (int)(th - t * H);
    const float s = sigmoid_exact(ldf(gate + t * gate_stride + h));
    float v[8];
    ld8(out + i * 8, v);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] *= s;
    st8(out + i * 8, v);
  }
}

// grid (T, 2), dynamic LDS (max(H, G) * D + 2R) floats. y = 0: the query row — RMS norm
// over the whole projection (H*D entries, one weight each), rotation of the
// first 2R entries of every head with entry i paired with i + R
// (angle = pos * inv_freq[i], fp32), written back in place. y = 1: the same for
// the key row into k_cache, and the value row into v_cache. The normed row is
// staged in LDS so that partners are read before anything is overwritten.
template <typename T>
__global__ void qk_fullnorm_rope_store_kernel(T* __restrict__ q, const T* __restrict__ k, const T* __restrict__ v,
                                              const float* __restrict__ wq, const float* __restrict__ wk,
                                              float eps, const int64_t* __restrict__ positions,
                                              const float* __restrict__ inv_freq, T* __restrict__ k_cache,
                                              T* __restrict__ v_cache, const int64_t* __restrict__ slots, int H,
                                              int G, int D, int Dv, int R, int BS, int q_stride, int k_stride,
                                              int v_stride) {
  extern __shared__ float nrow[];          // the normed row | cos [R] | sin [R]
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const bool is_q = blockIdx.y == 0;
  const int heads = is_q ? H : G;
  const int n = heads * D;
  const T* src = is_q ? q + (int64_t)t * q_stride : k + (int64_t)t * k_stride;
  const float* w = is_q ? wq : wk;
  float ss = 0.f;
  for (int i = threadIdx.x; i < n; i += blockDim.x) { const float x = ldf(src + i); nrow[i] = x; ss += x * x; }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)n + eps);
  for (int i = threadIdx.x; i < n; i += blockDim.x) nrow[i] *= r * w[i];
  const float pos = (float)positions[t];
  float* cs_t = nrow + n;
  float* sn_t = cs_t + R;
  for (int i = threadIdx.x; i < R; i += blockDim.x) sincosf(pos * inv_freq[i], &sn_t[i], &cs_t[i]);
  __syncthreads();
  int64_t blk = 0, off = 0;
  if (!is_q) { const int64_t slot = slots[t]; blk = slot / BS; off = slot % BS; }
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int h = i / D, d = i - h * D;
    float val = nrow[i];
    if (d < 2 * R) {
      const int f = d < R ? d : d - R;
      const float sn = sn_t[f], cs = cs_t[f];
      val = d < R ? val * cs - nrow[i + R] * sn : val * cs + nrow[i - R] * sn;
    }
    if (is_q) stf(q + (int64_t)t * q_stride + i, val);
    else stf(k_cache + ((blk * G + h) * BS + off) * D + d, val);
  }
  if (!is_q) {
    for (int i = threadIdx.x; i < G * Dv; i += blockDim.x) {
      const int g = i / Dv, d = i - g * Dv;
      v_cache[((blk * G + g) * BS + off) * Dv + d] = v[(int64_t)t * v_stride + i];
    }
  }
}

// grid (rows, G): a row whose position ends an aligned run of ``run`` positions
// writes the fp32 means of the run's cached keys and values into the pooled
// caches [NB, G, PB, D|Dv]; other rows leave at once. row_map (optional): the
// rows to look at — the host knows which rows of a prompt portion end a run. The run's tokens are
// found through the block table: some may date from earlier steps.
template <typename T>
__global__ void pool_kv_update_kernel(const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                                      float* __restrict__ pool_k, float* __restrict__ pool_v,
                                      const int* __restrict__ block_tables, const int* __restrict__ token_seg,
                                      const int64_t* __restrict__ positions, const int* __restrict__ row_map,
                                      int run, int PB, int G, int D, int Dv, int BS, int bt_stride) {
  const int t = row_map ? row_map[blockIdx.x] : blockIdx.x, g = blockIdx.y;
  const int p = (int)positions[t];
  if ((p + 1) % run != 0) return;
  const int b = p / run;
  const int* bt = block_tables + (int64_t)token_seg[t] * bt_stride;
  const int pg = p / BS;
  const int64_t prow = (int64_t)(bt[pg] * G + g) * PB + (b - (pg * BS) / run);
  const float inv = 1.0f / (float)run;
  for (int d = threadIdx.x; d < D + Dv; d += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < run; ++j) {
      const int pp = b * run + j;
      const int64_t row = (int64_t)(bt[pp / BS] * G + g) * BS + (pp % BS);
      acc += d < D ? ldf(k_cache + row * D + d) : ldf(v_cache + row * Dv + (d - D));
    }
    if (d < D) pool_k[prow * D + d] = acc * inv;
    else pool_v[prow * Dv + (d - D)] = acc * inv;
  }
}

// The same with 16-byte loads (D and Dv multiples of 8, (D + Dv) / 8 <= 256):
// LPP lanes cover one token's key and value row, the block's 256 / LPP lane
// groups take the run's tokens in turn, and their partial sums meet in LDS.
template <typename T>
__global__ void __launch_bounds__(256) pool_kv_update_v8_kernel(
    const T* __restrict__ k_cache, const T* __restrict__ v_cache, float* __restrict__ pool_k,
    float* __restrict__ pool_v, const int* __restrict__ block_tables, const int* __restrict__ token_seg,
    const int64_t* __restrict__ positions, const int* __restrict__ row_map, int run, int PB, int G, int D,
    int Dv, int BS, int bt_stride) {
  __shared__ float red[256 * 8];
  const int t = row_map ? row_map[blockIdx.x] : blockIdx.x, g = blockIdx.y;
  const int p = (int)positions[t];
  if ((p + 1) % run != 0) return;
  const int b = p / run;
  const int* bt = block_tables + (int64_t)token_seg[t] * bt_stride;
  const int pg = p / BS;
  const int64_t prow = (int64_t)(bt[pg] * G + g) * PB + (b - (pg * BS) / run);
  const int LPP = (D + Dv) / 8, NPG = 256 / LPP;
  const int dl = threadIdx.x % LPP, grp = threadIdx.x / LPP;
  const int d0 = dl * 8;
  float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  if (grp < NPG) {
    for (int j = grp; j < run; j += NPG) {
      const int pp = b * run + j;
      const int64_t row = (int64_t)(bt[pp / BS] * G + g) * BS + (pp % BS);
      float v[8];
      if (d0 < D) ld8(k_cache + row * D + d0, v);
      else ld8(v_cache + row * Dv + (d0 - D), v);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += v[e];
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[threadIdx.x * 8 + e] = acc[e];
  __syncthreads();
  if (grp == 0) {
    for (int g2 = 1; g2 < NPG; ++g2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += red[(g2 * LPP + dl) * 8 + e];
    }
    const float inv = 1.0f / (float)run;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] *= inv;
    if (d0 < D) st8(pool_k + prow * D + d0, acc);
    else st8(pool_v + prow * Dv + (d0 - D), acc);
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

extern "C" void seq_launch_rope_pairs_store(void* q, const void* k, const void* v, const int64_t* positions,
                                            const float* inv_freq, void* k_cache, void* v_cache,
                                            const int64_t* slots, void* kv_fresh, int T_, int H, int G, int D,
                                            int Dv, int R,
                                            int BS, int q_stride, int k_stride, int v_stride, int is_f32,
                                            hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(rope_pairs_store_kernel<T>, dim3(T_, H + G), dim3(WAVE), 0, st,
                                        (T*)q, (const T*)k, (const T*)v, positions, inv_freq, (T*)k_cache,
                                        (T*)v_cache, slots, (T*)kv_fresh, H, G, D, Dv, R, BS, q_stride, k_stride,
                                        v_stride);)
}

extern "C" void seq_launch_qk_norm_store(void* q, const void* k, const void* v, const float* wq,
                                         const float* wk, float eps, void* k_cache, void* v_cache,
                                         const int64_t* slots, int T_, int H, int G, int D, int Dv, int BS,
                                         int q_stride, int k_stride, int v_stride, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(qk_norm_store_kernel<T>, dim3(T_, H + G), dim3(WAVE), 0, st, (T*)q,
                                        (const T*)k, (const T*)v, wq, wk, eps, (T*)k_cache, (T*)v_cache, slots,
                                        H, G, D, Dv, BS, q_stride, k_stride, v_stride);)
}

extern "C" void seq_launch_attn_masked_paged(void* out, const void* q, const void* k_cache,
                                             const void* v_cache, const int* block_tables,
                                             const int* token_seg, const int64_t* positions,
                                             const void* gate, const int* row_map, int n_rows,
                                             const float* pool_k, const float* pool_v, int run, int PB,
                                             float softcap, int nsplit, float* part_o, float* part_ml,
                                             float scale, int mask_kind, int mask_size, int keep_first,
                                             int sink, int gate_kind, int T_, int H,
                                             int G, int D, int Dv, int BS, int bt_stride, int q_stride,
                                             int gate_stride, int is_f32, hipStream_t st) {
  const size_t lds = (size_t)(D + 2 * WAVE) * sizeof(float);
  const int rows = row_map ? n_rows : T_;
  const int lpk = D / 8, lpv = Dv / 8;
  if (D % 8 == 0 && Dv % 8 == 0 && lpk <= 64 && lpv <= 64 && (lpk & (lpk - 1)) == 0 && (lpv & (lpv - 1)) == 0 &&
      q_stride % 8 == 0 && aligned16(q) && aligned16(k_cache) && aligned16(v_cache) && aligned16(out) &&
      (gate_kind != 2 || (gate_stride % 8 == 0 && aligned16(gate))) &&
      (pool_k == nullptr || (aligned16(pool_k) && aligned16(pool_v)))) {
    // key shares only for plain launches: every row, no gate
    const int ns = (nsplit > 1 && row_map == nullptr && gate_kind == 0 && part_o != nullptr) ? nsplit : 1;
    DISPATCH_T(is_f32, hipLaunchKernelGGL(attn_blocklocal_paged_v8_kernel<T>, dim3(rows, H, ns), dim3(WAVE * ATTN_V8_WAVES), 0, st,
                                          (T*)out, (const T*)q, (const T*)k_cache, (const T*)v_cache,
                                          block_tables, token_seg, positions, (const T*)gate, row_map, pool_k,
                                          pool_v, run, PB, softcap, part_o, part_ml, scale,
                                          mask_kind, mask_size, keep_first, sink, gate_kind, H, G, D, Dv, BS,
                                          bt_stride, q_stride, gate_stride);)
    if (ns > 1) {
      const int threads = Dv / 8 > WAVE ? 2 * WAVE : WAVE;
      DISPATCH_T(is_f32, hipLaunchKernelGGL(attn_split_merge_kernel<T>, dim3(rows, H), dim3(threads), 0, st,
                                            (T*)out, part_o, part_ml, H, Dv, ns);)
    }
    return;
  }
  DISPATCH_T(is_f32, hipLaunchKernelGGL(attn_blocklocal_paged_kernel<T>, dim3(rows, H), dim3(WAVE), lds, st,
                                        (T*)out, (const T*)q, (const T*)k_cache, (const T*)v_cache,
                                        block_tables, token_seg, positions, (const T*)gate, row_map, pool_k,
                                        pool_v, run, PB, softcap, scale,
                                        mask_kind, mask_size, keep_first, sink, gate_kind,
                                        H, G, D, Dv, BS, bt_stride, q_stride, gate_stride);)
}

extern "C" void seq_launch_head_gate(void* out, const void* gate, int T_, int H, int Dv, int gate_stride,
                                     int is_f32, hipStream_t st) {
  const int64_t n = (int64_t)T_ * H * Dv;
  if (Dv % 8 == 0 && aligned16(out)) {
    const int g8 = (int)((n / 8 + 255) / 256 < 16384 ? (n / 8 + 255) / 256 : 16384);
    DISPATCH_T(is_f32, hipLaunchKernelGGL(head_gate_v8_kernel<T>, dim3(g8), dim3(256), 0, st, (T*)out,
                                          (const T*)gate, n / 8, H, Dv / 8, gate_stride);)
    return;
  }
  const int grid = (int)((n + 255) / 256 < 8192 ? (n + 255) / 256 : 8192);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(head_gate_kernel<T>, dim3(grid), dim3(256), 0, st, (T*)out,
                                        (const T*)gate, n, H, Dv, gate_stride);)
}

extern "C" void seq_launch_qk_fullnorm_rope_store(void* q, const void* k, const void* v, const float* wq,
                                                  const float* wk, float eps, const int64_t* positions,
                                                  const float* inv_freq, void* k_cache, void* v_cache,
                                                  const int64_t* slots, int T_, int H, int G, int D, int Dv,
                                                  int R, int BS, int q_stride, int k_stride, int v_stride,
                                                  int is_f32, hipStream_t st) {
  const int heads = H > G ? H : G;
  const size_t lds = ((size_t)heads * D + 2 * R) * sizeof(float);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(qk_fullnorm_rope_store_kernel<T>, dim3(T_, k != nullptr ? 2 : 1),
                                        dim3(256), lds, st, (T*)q, (const T*)k, (const T*)v, wq, wk, eps,
                                        positions, inv_freq, (T*)k_cache, (T*)v_cache, slots, H, G, D, Dv, R, BS,
                                        q_stride, k_stride, v_stride);)
}

extern "C" void seq_launch_pool_kv_update(const void* k_cache, const void* v_cache, float* pool_k, float* pool_v,
                                          const int* block_tables, const int* token_seg,
                                          const int64_t* positions, const int* row_map, int run, int PB, int T_,
                                          int G, int D, int Dv, int BS, int bt_stride, int is_f32,
                                          hipStream_t st) {
  if (D % 8 == 0 && Dv % 8 == 0 && (D + Dv) / 8 <= 256 && aligned16(k_cache) && aligned16(v_cache) &&
      aligned16(pool_k) && aligned16(pool_v)) {
    DISPATCH_T(is_f32, hipLaunchKernelGGL(pool_kv_update_v8_kernel<T>, dim3(T_, G), dim3(256), 0, st,
                                          (const T*)k_cache, (const T*)v_cache, pool_k, pool_v, block_tables,
                                          token_seg, positions, row_map, run, PB, G, D, Dv, BS, bt_stride);)
    return;
  }
  const int threads = D + Dv > 128 ? 256 : (D + Dv > 64 ? 128 : 64);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(pool_kv_update_kernel<T>, dim3(T_, G), dim3(threads), 0, st,
                                        (const T*)k_cache, (const T*)v_cache, pool_k, pool_v, block_tables,
                                        token_seg, positions, row_map, run, PB, G, D, Dv, BS, bt_stride);)
}
