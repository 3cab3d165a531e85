// Latent attention: every token caches ONE row [latent c (C) | rotated key
// part (R)] that all heads share. In the absorbed form a head's query is
// [W_uk^T q_unrotated (C) | q_rotated (R)], its score against token j is the
// dot product with j's cached row, and its output is the weighted sum of the
// latents (W_uv is applied afterwards). The kernels here:
//   latent_kv_store    query rotation in place, latent RMS norm, key-part
//                      rotation, paged store of the cached row (one launch)
//   attn_latent_paged  sliding-window softmax attention over the paged rows
//     - a plain kernel (any size, bf16 or fp32; the exact-mode path)
//     - an MFMA kernel (bf16): 32 (row, head) query columns of one workgroup
//       share each staged tile of 32 cached rows, for prompt portions,
//       decoded tokens and mixes alike.
// Scores, softmax weights and the running sums are fp32 everywhere.

#include "seq_common.h"

// ---- step input ----------------------------------------------------------------
// One workgroup of 256 threads per row. All threads: rotate the last R entries of
// every query head (interleaved pairs, angle = float(pos) * inv_freq[i]) in
// place. Then the row's down-projection dkv [C + R] -> cache row
// [rms(dkv[:C]) * w | rotate(dkv[C:])].
template <typename T>
__global__ void __launch_bounds__(256) latent_kv_store_kernel(
    T* __restrict__ q, const T* __restrict__ dkv, const float* __restrict__ w, float eps,
    const int64_t* __restrict__ positions, const float* __restrict__ inv_freq, T* __restrict__ cache,
    const int64_t* __restrict__ slots, int H, int D, int R, int C, int q_stride, int dkv_stride) {
  __shared__ float scratch[16];
  const int t = blockIdx.x, tid = threadIdx.x;
  const float pos = (float)positions[t];
  const int R2 = R / 2;
  const T* src = dkv + (int64_t)t * dkv_stride;
  T* dst = cache + slots[t] * (int64_t)(C + R);
  float ss = 0.f;
  for (int i = tid; i < C; i += blockDim.x) { const float x = ldf(src + i); ss += x * x; }
  T* qrow = q + (int64_t)t * q_stride + D;
  for (int idx = tid; idx < H * R2; idx += blockDim.x) {
    const int h = idx / R2, i = idx - h * R2;
    T* row = qrow + (int64_t)h * (D + R);
    float s, c;
    sincosf(pos * inv_freq[i], &s, &c);
    const float u = ldf(row + 2 * i), v = ldf(row + 2 * i + 1);
    stf(row + 2 * i, u * c - v * s);
    stf(row + 2 * i + 1, v * c + u * s);
  }
  ss = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(ss / (float)C + eps);
  for (int i = tid; i < C; i += blockDim.x) stf(dst + i, ldf(src + i) * r * w[i]);
  for (int i = tid; i < R2; i += blockDim.x) {
    float s, c;
    sincosf(pos * inv_freq[i], &s, &c);
    const float u = ldf(src + C + 2 * i), v = ldf(src + C + 2 * i + 1);
    stf(dst + C + 2 * i, u * c - v * s);
    stf(dst + C + 2 * i + 1, v * c + u * s);
  }
}

// ---- plain attention kernel ------------------------------------------------------
// grid (T, H), one wave per (query row, head). Visible keys lo..p in tiles of
// 64: lane u scores key lo + tile*64 + u against the query staged in LDS, the
// tile's weights go through LDS, then lanes own output dims and sweep the
// tile's latent rows. Online softmax in fp32.
#define LAT_MAX_ACC 16   // C <= 1024
template <typename T>
__global__ void attn_latent_paged_kernel(T* __restrict__ out, const T* __restrict__ q_abs,
                                         const T* __restrict__ q, const T* __restrict__ cache,
                                         const int* __restrict__ block_tables,
                                         const int* __restrict__ token_seg,
                                         const int64_t* __restrict__ positions, const T* __restrict__ gate,
                                         float scale, int mask_size, int H, int D, int R, int C, int BS,
                                         int bt_stride, int64_t qa_stride_t, int64_t qa_stride_h, int q_stride,
                                         int gate_stride) {
  extern __shared__ float lds[];       // query [C + R] | weights [64] | cache row index [64] (as int)
  const int L = C + R;
  float* qs = lds;
  float* ps = lds + L;
  int* rows = (int*)(ps + WAVE);
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int p = (int)positions[t];
  const int lo = mask_size > 0 ? max(0, p - mask_size + 1) : 0;
  const int total = p - lo + 1;
  const int* bt = block_tables + (int64_t)token_seg[t] * bt_stride;
  const T* qa = q_abs + t * qa_stride_t + h * qa_stride_h;
  const T* qr = q + (int64_t)t * q_stride + (int64_t)h * (D + R) + D;
  for (int i = lane; i < C; i += WAVE) qs[i] = ldf(qa + i) * scale;
  for (int i = lane; i < R; i += WAVE) qs[C + i] = ldf(qr + i) * scale;
  __syncthreads();

  float acc[LAT_MAX_ACC];
#pragma unroll
  for (int i = 0; i < LAT_MAX_ACC; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int base = 0; base < total; base += WAVE) {
    const int u = base + lane;
    float s = -INFINITY;
    int row = -1;
    if (u < total) {
      const int j = lo + u;
      row = bt[j / BS] * BS + (j % BS);
      const T* kr = cache + (int64_t)row * L;
      float d = 0.f;
      for (int i = 0; i < L; ++i) d += qs[i] * ldf(kr + i);
      s = d;
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
    for (int i = 0; i < LAT_MAX_ACC; ++i) acc[i] *= corr;
    for (int jj = 0; jj < n; ++jj) {
      const float pw = ps[jj];
      const T* vr = cache + (int64_t)rows[jj] * L;
#pragma unroll
      for (int i = 0; i < LAT_MAX_ACC; ++i) {
        const int d = lane + i * WAVE;
        if (d < C) acc[i] += pw * ldf(vr + d);
      }
    }
    __syncthreads();
  }
  float gsc = 1.0f / l;
  if (gate != nullptr) gsc *= sigmoid_exact(ldf(gate + (int64_t)t * gate_stride + h));
  T* orow = out + ((int64_t)t * H + h) * C;
#pragma unroll
  for (int i = 0; i < LAT_MAX_ACC; ++i) {
    const int d = lane + i * WAVE;
    if (d < C) stf(orow + d, acc[i] * gsc);
  }
}

// ---- MFMA attention kernel (bf16) ---------------------------------------------------
// v_mfma_f32_32x32x16_bf16 fragment maps:
//   A[i][k]: lane l holds i = l&31, k = (l>>5)*8 + j   (j = 0..7)
//   B[k][j]: lane l holds j = l&31, k = (l>>5)*8 + jj
//   C[i][j]: lane l holds j = l&31, i = (r&3) + 8*(r>>2) + 4*(l>>5)  (r = 0..15)
//
// A workgroup of 4 waves serves one tile of `tile_rows` consecutive packed
// rows x `hb` heads = up to 32 query columns (column c = row c / hb, head
// h0 + c % hb). Rows of a tile that belong to different sequences are served
// in turn (one pass over the keys per sequence present in the tile; columns of
// other sequences are masked out of the pass). With single-row tiles (steps of
// decoded tokens) gridDim.z workgroups take contiguous shares of the row's key
// tiles and leave unnormalised partial results (sums, running max and sum)
// that attn_latent_merge_kernel combines in a fixed order.
//
// Per tile of 32 keys:
//   all threads stage the 32 cached rows [32][Lp] (zero-padded to a multiple
//   of 16 dims) in LDS; the next tile's rows are already on their way from
//   memory while the current tile is worked on;
//   S^T[key][col] = rows x query^T: the 16-dim slices of the dot product are
//   dealt round-robin to the waves, each writes its partial S^T to LDS and
//   every wave sums the four partials in the same order (so all waves hold
//   identical scores);
//   mask, scale, online softmax: a column's 32 scores sit in one lane pair
//   (l, l ^ 32), the rest is lane-local;
//   O^T[d][col] += latent^T x P: the 32-dim output tiles are dealt
//   round-robin to the waves. P enters the matrix unit as a sum of two bf16
//   parts (the rounding of p and the rounding of what that left), so the
//   weights keep 16 bits of mantissa; the latent fragments are read from the
//   staged rows by columns.
typedef __bf16 lat_bf16x8 __attribute__((ext_vector_type(8)));
typedef float lat_f32x16 __attribute__((ext_vector_type(16)));

#define LAT_WAVES 4
#define LAT_KT 32            // keys per tile
#define LAT_MAX_SL 9         // 16-dim slices per wave: C + R <= 576
#define LAT_MAX_DT 4         // 32-dim output tiles per wave: C <= 512
#define LAT_PAD 8            // bf16 elements of padding per staged row
#define LAT_STAGE 9          // 16-byte chunks per staging thread: 8 threads per row, rows up to 576 wide

__device__ __forceinline__ int lat_acc_row(int r, int half) { return (r & 3) + 8 * (r >> 2) + 4 * half; }

typedef float lat_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 lat_bf16x2 __attribute__((ext_vector_type(2)));

// two floats -> two bf16 (round to nearest even) packed in one word, low half first
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const lat_f32x2 v = {a, b};
  lat_bf16x2 r = __builtin_convertvector(v, lat_bf16x2);
  return *reinterpret_cast<uint32_t*>(&r);
}

// Workgroup barrier that orders LDS traffic only: every wave's LDS reads and
// writes are complete (lgkmcnt 0) before it arrives, global loads in flight
// stay in flight. The tile loop prefetches the next tile's rows into
// registers, and a full __syncthreads would wait for them at every barrier.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt(0xc07f);      // vmcnt 63, expcnt 7, lgkmcnt 0
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__global__ void __launch_bounds__(WAVE * LAT_WAVES, 2) attn_latent_mfma_kernel(
    bfraw* __restrict__ out, const bfraw* __restrict__ q_abs, const bfraw* __restrict__ q,
    const bfraw* __restrict__ cache, const int* __restrict__ block_tables, const int* __restrict__ token_seg,
    const int64_t* __restrict__ positions, const bfraw* __restrict__ gate, float scale, int mask_size, int T_,
    int H, int D, int R, int C, int BS, int bt_stride, int64_t qa_stride_t, int64_t qa_stride_h, int q_stride,
    int gate_stride, int tile_rows, int hb, int vec, int qvec, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  extern __shared__ __align__(16) unsigned char lat_smem[];
  const int L = C + R;
  const int Lp = (L + 15) / 16 * 16;
  const int kstride = Lp + LAT_PAD;                       // staged row stride in elements
  bfraw* k_lds = reinterpret_cast<bfraw*>(lat_smem);                                   // [32][kstride]
  float* s_lds = reinterpret_cast<float*>(lat_smem + (size_t)LAT_KT * kstride * 2);    // [4][16][64]

  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int half = lane >> 5, col = lane & 31;
  const int skey = tid >> 3, spart = tid & 7;              // staging role
  const int row0 = blockIdx.x * tile_rows;
  const int h0 = blockIdx.y * hb;
  const int nrows = min(tile_rows, T_ - row0);
  // this lane's query column
  const int crow = col / hb, chead = h0 + col % hb;
  const bool cvalid = crow < nrows && chead < H;
  const int ct = row0 + (cvalid ? crow : 0);
  const int cpos = (int)positions[ct];
  const int cseg = token_seg[ct];
  const int clo = mask_size > 0 ? max(0, cpos - mask_size + 1) : 0;

  // query fragments (B operand) of this wave's slices: dims s*16 + half*8 + jj.
  // The 32 columns' query rows [C | R] go through the (not yet used) key
  // buffer: thread (skey, spart) loads chunks of column skey, then every lane
  // reads its fragments back with 16-byte LDS loads.
  const int nslice = Lp / 16;
  lat_bf16x8 q_frag[LAT_MAX_SL];
  {
    const int srow = skey / hb, shead = h0 + skey % hb;
    const bool sval = srow < nrows && shead < H;
    const int st_ = row0 + (sval ? srow : 0);
    const bfraw* qa = q_abs + st_ * qa_stride_t + (sval ? shead : 0) * qa_stride_h;
    const bfraw* qr = q + (int64_t)st_ * q_stride + (int64_t)(sval ? shead : 0) * (D + R) + D;
    uint4 qst[LAT_STAGE];
#pragma unroll
    for (int i = 0; i < LAT_STAGE; ++i) {
      const int c8 = (spart + 8 * i) * 8;
      uint4 val = make_uint4(0, 0, 0, 0);
      if (sval && c8 < L) {
        if (qvec && c8 + 8 <= L) {                       // C % 8 == 0: a chunk lies in one of the two parts
          val = *reinterpret_cast<const uint4*>(c8 < C ? qa + c8 : qr + (c8 - C));
        } else {
          __attribute__((aligned(16))) bfraw e[8];
#pragma unroll
          for (int jj = 0; jj < 8; ++jj) {
            const int d = c8 + jj;
            e[jj] = d < L ? (d < C ? qa[d] : qr[d - C]) : (bfraw)0;
          }
          val = *reinterpret_cast<uint4*>(e);
        }
      }
      qst[i] = val;
    }
#pragma unroll
    for (int i = 0; i < LAT_STAGE; ++i) {
      const int c8 = (spart + 8 * i) * 8;
      if (c8 < Lp) *reinterpret_cast<uint4*>(k_lds + skey * kstride + c8) = qst[i];
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < LAT_MAX_SL; ++i) {
      const int s = wave + i * LAT_WAVES;
      if (s < nslice) q_frag[i] = *reinterpret_cast<const lat_bf16x8*>(k_lds + col * kstride + s * 16 + half * 8);
    }
    __syncthreads();
  }

  const int ndt = (C + 31) / 32;
  lat_f32x16 o_acc[LAT_MAX_DT];
#pragma unroll
  for (int i = 0; i < LAT_MAX_DT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) o_acc[i][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float scale2 = scale * 1.4426950408889634f;

  // one pass per sequence present in the tile (rows are packed by sequence)
  int ra = 0;
  while (ra < nrows) {
    const int seg = token_seg[row0 + ra];
    int rb = ra + 1;
    while (rb < nrows && token_seg[row0 + rb] == seg) ++rb;
    const int p_first = (int)positions[row0 + ra], p_last = (int)positions[row0 + rb - 1];
    const int key_lo = mask_size > 0 ? max(0, p_first - mask_size + 1) : 0;
    const int* bt = block_tables + (int64_t)seg * bt_stride;
    const bool mine = cvalid && cseg == seg && crow >= ra && crow < rb;
    // gridDim.z > 1 (single-row tiles only): this workgroup takes a contiguous
    // share of the row's key tiles and leaves an unnormalised partial result
    int k_begin = key_lo, k_last = p_last;
    if (gridDim.z > 1) {
      const int ntiles = (p_last - key_lo) / LAT_KT + 1;
      const int tps = (ntiles + gridDim.z - 1) / gridDim.z;
      k_begin = key_lo + (int)blockIdx.z * tps * LAT_KT;
      k_last = min(p_last, k_begin + tps * LAT_KT - 1);
    }

    // Staging: thread (skey, spart) of the 32 x 8 grid loads the 16-byte chunks
    // spart, spart + 8, ... of cached row skey. The loads of the NEXT tile are
    // issued before the current tile is worked on and land in LDS after it.
    uint4 stage[LAT_STAGE];
    auto fetch = [&](int kt0) {
      const int nk = min(LAT_KT, k_last - kt0 + 1);
      const int j = kt0 + min(skey, nk - 1);
      const bfraw* src = cache + (int64_t)(bt[j / BS] * BS + (j % BS)) * L;
#pragma unroll
      for (int i = 0; i < LAT_STAGE; ++i) {
        const int c8 = (spart + 8 * i) * 8;
        uint4 val = make_uint4(0, 0, 0, 0);
        if (skey < nk && c8 < Lp) {
          if (vec && c8 + 8 <= L) {
            val = *reinterpret_cast<const uint4*>(src + c8);
          } else {
            __attribute__((aligned(16))) bfraw e[8];
#pragma unroll
            for (int jj = 0; jj < 8; ++jj) e[jj] = c8 + jj < L ? src[c8 + jj] : (bfraw)0;
            val = *reinterpret_cast<uint4*>(e);
          }
        }
        stage[i] = val;
      }
    };
    if (k_begin <= k_last) fetch(k_begin);
    for (int kt0 = k_begin; kt0 <= k_last; kt0 += LAT_KT) {
      const int nkeys = min(LAT_KT, k_last - kt0 + 1);
#pragma unroll
      for (int i = 0; i < LAT_STAGE; ++i) {
        const int c8 = (spart + 8 * i) * 8;
        if (c8 < Lp) *reinterpret_cast<uint4*>(k_lds + skey * kstride + c8) = stage[i];
      }
      lds_barrier();
      if (kt0 + LAT_KT <= k_last) fetch(kt0 + LAT_KT);
      // ---- partial S^T over this wave's slices ---------------------------------
      {
        lat_f32x16 s_acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) s_acc[r] = 0.f;
#pragma unroll
        for (int i = 0; i < LAT_MAX_SL; ++i) {
          const int s = wave + i * LAT_WAVES;
          if (s < nslice) {
            const lat_bf16x8 a = *reinterpret_cast<const lat_bf16x8*>(k_lds + col * kstride + s * 16 + half * 8);
            s_acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, q_frag[i], s_acc, 0, 0, 0);
          }
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) s_lds[(wave * 16 + r) * WAVE + lane] = s_acc[r];
      }
      lds_barrier();
      float sv[16];
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float a = s_lds[r * WAVE + lane];
#pragma unroll
        for (int w2 = 1; w2 < LAT_WAVES; ++w2) a += s_lds[(w2 * 16 + r) * WAVE + lane];
        const int kk = lat_acc_row(r, half);
        const int key = kt0 + kk;
        const bool ok = mine && kk < nkeys && key <= cpos && key >= clo;
        sv[r] = ok ? a * scale2 : -INFINITY;            // scores in units of ln 2: weights are 2^(s - m)
      }
      // ---- online softmax; a column's scores sit in lanes l and l ^ 32 -----------
      float tmax = sv[0];
#pragma unroll
      for (int r = 1; r < 16; ++r) tmax = fmaxf(tmax, sv[r]);
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
      const float m_new = fmaxf(m_run, tmax);
      const float m_ref = m_new == -INFINITY ? 0.f : m_new;      // nothing seen yet: every weight below is 2^-inf = 0
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_ref);
      m_run = m_new;
      float p[16], psum = 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        p[r] = __builtin_amdgcn_exp2f(sv[r] - m_ref);
        psum += p[r];
      }
      l_run = l_run * alpha + psum;
      if (__builtin_amdgcn_ballot_w64(alpha != 1.0f)) {           // the running maximum moved in some column
#pragma unroll
        for (int i = 0; i < LAT_MAX_DT; ++i)
#pragma unroll
          for (int r = 0; r < 16; ++r) o_acc[i][r] *= alpha;
      }
      // ---- P as two bf16 parts, repacked into B fragments --------------------------
      // B[k][j]: lane (j, hf) needs keys kt*16 + hf*8 + 0..7 of column j. Lane
      // (j, half) holds keys lat_acc_row(r, half): r = 4g + i -> key 8g + 4*half + i.
      // Fragment kt of lane (j, hf) = keys 16kt + 8hf + {0..3} from lane (j, 0),
      // regs 4(2kt + hf) + {0..3}, and {4..7} from lane (j, 1), the same regs.
      uint32_t hi2[8], lo2[8];
#pragma unroll
      for (int pr = 0; pr < 8; ++pr) {
        hi2[pr] = pack_bf16x2(p[2 * pr], p[2 * pr + 1]);
        union { uint32_t u; float f; } c0, c1;
        c0.u = hi2[pr] << 16; c1.u = hi2[pr] & 0xffff0000u;
        lo2[pr] = pack_bf16x2(p[2 * pr] - c0.f, p[2 * pr + 1] - c1.f);
      }
      lat_bf16x8 pf_hi[2], pf_lo[2];
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        // group g = 2kt + hf: words 2g, 2g+1 of the lane with half 0, then of the lane with half 1
        __attribute__((aligned(16))) uint32_t wh[4], wl[4];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
          const int g = 2 * kt + hf;
          // what the partner lane (other half) holds for group g
          const uint32_t oh0 = __shfl_xor(hi2[2 * g], 32), oh1 = __shfl_xor(hi2[2 * g + 1], 32);
          const uint32_t ol0 = __shfl_xor(lo2[2 * g], 32), ol1 = __shfl_xor(lo2[2 * g + 1], 32);
          if (hf == half) {
            // this lane builds its own fragment from group g: keys 0..3 from half 0, 4..7 from half 1
            wh[0] = half == 0 ? hi2[2 * g] : oh0;  wh[1] = half == 0 ? hi2[2 * g + 1] : oh1;
            wh[2] = half == 0 ? oh0 : hi2[2 * g];  wh[3] = half == 0 ? oh1 : hi2[2 * g + 1];
            wl[0] = half == 0 ? lo2[2 * g] : ol0;  wl[1] = half == 0 ? lo2[2 * g + 1] : ol1;
            wl[2] = half == 0 ? ol0 : lo2[2 * g];  wl[3] = half == 0 ? ol1 : lo2[2 * g + 1];
          }
        }
        pf_hi[kt] = *reinterpret_cast<lat_bf16x8*>(wh);
        pf_lo[kt] = *reinterpret_cast<lat_bf16x8*>(wl);
      }
      // ---- O^T += latent^T x P over this wave's output tiles ------------------------
#pragma unroll
      for (int i = 0; i < LAT_MAX_DT; ++i) {
        const int dt = wave + i * LAT_WAVES;
        if (dt < ndt) {
          const int d = dt * 32 + col;            // < Lp: columns beyond C hold the key part or zeros, never stored
#pragma unroll
          for (int kt = 0; kt < 2; ++kt) {
            __attribute__((aligned(16))) bfraw e[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) e[j] = k_lds[(kt * 16 + half * 8 + j) * kstride + min(d, Lp - 1)];
            const lat_bf16x8 a = *reinterpret_cast<lat_bf16x8*>(e);
            o_acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf_hi[kt], o_acc[i], 0, 0, 0);
            o_acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pf_lo[kt], o_acc[i], 0, 0, 0);
          }
        }
      }
      lds_barrier();
    }
    ra = rb;
  }

  // ---- epilogue: the column's two half sums, 1/l, gate, store ------------------------
  l_run += __shfl_xor(l_run, 32);
  if (gridDim.z > 1) {
    // partial result of this key share: [T, H, splits, C] sums and (max, sum) in units of ln 2
    if (cvalid) {
      const int64_t slot = ((int64_t)ct * H + chead) * gridDim.z + blockIdx.z;
      if (wave == 0 && half == 0) { part_ml[2 * slot] = m_run; part_ml[2 * slot + 1] = l_run; }
      float* po = part_o + slot * C;
#pragma unroll
      for (int i = 0; i < LAT_MAX_DT; ++i) {
        const int dt = wave + i * LAT_WAVES;
        if (dt < ndt) {
#pragma unroll
          for (int g4 = 0; g4 < 4; ++g4) {             // regs 4 g4 .. 4 g4 + 3 hold 4 consecutive dims
            const int d = dt * 32 + 8 * g4 + 4 * half;
            if (C % 4 == 0 && d + 4 <= C) {
              *reinterpret_cast<float4*>(po + d) = make_float4(o_acc[i][4 * g4], o_acc[i][4 * g4 + 1],
                                                               o_acc[i][4 * g4 + 2], o_acc[i][4 * g4 + 3]);
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (d + e < C) po[d + e] = o_acc[i][4 * g4 + e];
            }
          }
        }
      }
    }
    return;
  }
  if (cvalid) {
    float gsc = l_run > 0.f ? 1.0f / l_run : 0.f;
    if (gate != nullptr) gsc *= sigmoid_exact(ldf(gate + (int64_t)ct * gate_stride + chead));
    bfraw* orow = out + ((int64_t)ct * H + chead) * C;
    const bool ovec = C % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0;
#pragma unroll
    for (int i = 0; i < LAT_MAX_DT; ++i) {
      const int dt = wave + i * LAT_WAVES;
      if (dt < ndt) {
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {               // regs 4 g4 .. 4 g4 + 3 hold 4 consecutive dims
          const int d = dt * 32 + 8 * g4 + 4 * half;
          if (ovec && d + 4 <= C) {
            uint2 wd;
            wd.x = pack_bf16x2(o_acc[i][4 * g4] * gsc, o_acc[i][4 * g4 + 1] * gsc);
            wd.y = pack_bf16x2(o_acc[i][4 * g4 + 2] * gsc, o_acc[i][4 * g4 + 3] * gsc);
            *reinterpret_cast<uint2*>(orow + d) = wd;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (d + e < C) stf(orow + d + e, o_acc[i][4 * g4 + e] * gsc);
          }
        }
      }
    }
  }
}

// Merge of the key shares' partial results: grid (T, H), 256 threads. Every
// thread derives the shares' common maximum; the shares' factors 2^(m_z - M)
// go through LDS; threads own output dims and sum the shares in a fixed order.
#define LAT_MAX_SPLIT 64
__global__ void __launch_bounds__(256) attn_latent_merge_kernel(
    bfraw* __restrict__ out, const float* __restrict__ part_o, const float* __restrict__ part_ml,
    const bfraw* __restrict__ gate, int H, int C, int nsplit, int gate_stride) {
  __shared__ float fz[LAT_MAX_SPLIT];
  __shared__ float lsum;
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int64_t base = ((int64_t)t * H + h) * nsplit;
  float M = -INFINITY;
  for (int z = 0; z < nsplit; ++z) M = fmaxf(M, part_ml[2 * (base + z)]);
  if (tid < nsplit) {
    const float l = part_ml[2 * (base + tid) + 1];
    fz[tid] = l > 0.f ? __builtin_amdgcn_exp2f(part_ml[2 * (base + tid)] - M) : 0.f;
  }
  __syncthreads();
  if (tid == 0) {
    float L = 0.f;
    for (int z = 0; z < nsplit; ++z) L += part_ml[2 * (base + z) + 1] * fz[z];
    lsum = L;
  }
  __syncthreads();
  float gsc = lsum > 0.f ? 1.0f / lsum : 0.f;
  if (gate != nullptr) gsc *= sigmoid_exact(ldf(gate + (int64_t)t * gate_stride + h));
  for (int d = tid; d < C; d += 256) {
    const float* po = part_o + base * C + d;
    float acc = 0.f;
#pragma unroll 4
    for (int z = 0; z < nsplit; ++z) acc += po[(int64_t)z * C] * fz[z];
    stf(out + ((int64_t)t * H + h) * C + d, acc * gsc);
  }
}

#define DISPATCH_T(is_f32, ...)                                  \
  if (is_f32) { typedef float T; __VA_ARGS__ } else { typedef bfraw T; __VA_ARGS__ }

extern "C" void seq_launch_latent_kv_store(void* q, const void* dkv, const float* w, float eps,
                                           const int64_t* positions, const float* inv_freq, void* cache,
                                           const int64_t* slots, int T_, int H, int D, int R, int C,
                                           int q_stride, int dkv_stride, int is_f32, hipStream_t st) {
  DISPATCH_T(is_f32, hipLaunchKernelGGL(latent_kv_store_kernel<T>, dim3(T_), dim3(256), 0, st, (T*)q,
                                        (const T*)dkv, w, eps, positions, inv_freq, (T*)cache, slots, H, D, R, C,
                                        q_stride, dkv_stride);)
}

// tile_rows: rows per workgroup of the MFMA kernel (0 = as many as fit 32
// columns); use_mfma 0 forces the plain kernel. part_o [T, H, nsplit, C] /
// part_ml [T, H, nsplit, 2] (fp32, optional): with single-row tiles the keys of
// a row are shared out to nsplit workgroups and merged by a second kernel.
extern "C" void seq_launch_attn_latent_paged(void* out, const void* q_abs, const void* q, const void* cache,
                                             const int* block_tables, const int* token_seg,
                                             const int64_t* positions, const void* gate, float scale,
                                             int mask_size, int T_, int H, int D, int R, int C, int BS,
                                             int bt_stride, int64_t qa_stride_t, int64_t qa_stride_h,
                                             int q_stride, int gate_stride, int tile_rows, int use_mfma,
                                             float* part_o, float* part_ml, int nsplit, int is_f32,
                                             hipStream_t st) {
  const int L = C + R;
  if (use_mfma && !is_f32 && L <= 16 * LAT_WAVES * LAT_MAX_SL && C <= 32 * LAT_WAVES * LAT_MAX_DT) {
    int hb = 1;
    while (hb < H && hb < 32) hb <<= 1;                  // heads per tile: a power of two <= 32
    const int max_rows = 32 / hb;
    const int tr = tile_rows > 0 && tile_rows < max_rows ? tile_rows : max_rows;
    const int Lp = (L + 15) / 16 * 16;
    const size_t lds = (size_t)LAT_KT * (Lp + LAT_PAD) * 2 + (size_t)LAT_WAVES * 16 * WAVE * 4;
    const int vec = (L % 8 == 0 && aligned16(cache)) ? 1 : 0;
    const int qvec = (C % 8 == 0 && D % 8 == 0 && R % 8 == 0 && q_stride % 8 == 0 && qa_stride_t % 8 == 0 &&
                      qa_stride_h % 8 == 0 && aligned16(q) && aligned16(q_abs)) ? 1 : 0;
    const int ns = (tr == 1 && part_o != nullptr && nsplit > 1) ? nsplit : 1;
    hipLaunchKernelGGL(attn_latent_mfma_kernel, dim3((T_ + tr - 1) / tr, (H + hb - 1) / hb, ns),
                       dim3(WAVE * LAT_WAVES), lds, st, (bfraw*)out, (const bfraw*)q_abs, (const bfraw*)q,
                       (const bfraw*)cache, block_tables, token_seg, positions, (const bfraw*)gate, scale,
                       mask_size, T_, H, D, R, C, BS, bt_stride, qa_stride_t, qa_stride_h, q_stride, gate_stride,
                       tr, hb, vec, qvec, part_o, part_ml);
    if (ns > 1)
      hipLaunchKernelGGL(attn_latent_merge_kernel, dim3(T_, H), dim3(256), 0, st, (bfraw*)out, part_o, part_ml,
                         (const bfraw*)gate, H, C, ns, gate_stride);
    return;
  }
  const size_t lds = (size_t)(L + 2 * WAVE) * sizeof(float);
  DISPATCH_T(is_f32, hipLaunchKernelGGL(attn_latent_paged_kernel<T>, dim3(T_, H), dim3(WAVE), lds, st, (T*)out,
                                        (const T*)q_abs, (const T*)q, (const T*)cache, block_tables, token_seg,
                                        positions, (const T*)gate, scale, mask_size, H, D, R, C, BS, bt_stride,
                                        qa_stride_t, qa_stride_h, q_stride, gate_stride);)
}
