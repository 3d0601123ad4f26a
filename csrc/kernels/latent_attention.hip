// Latent (low-rank KV) attention over a paged latent cache.
//
// Cache row of one token: [ c (kv_rank, RMS-normed latent) | k_rot (rot_dim, rotated key part
// shared by all heads) ].  With the key up-projection absorbed into the query,
//   q_abs[h] = W_uk[h]^T q_nope[h]                       (a batched GEMM, done by the caller)
//   score[h][j] = (q_abs[h] . c_j + rot(q_rot[h]) . k_rot_j) * scale
//   lat[h] = sum_j softmax(score[h])_j c_j                (value up-projection by the caller)
// every head reads the SAME cache rows, so a workgroup stages a key tile in LDS once and uses it
// for all (query, head) rows it owns.  Scores, softmax weights and the accumulators are fp32;
// activations are bf16 or fp32 (template T).
//
//   eia_latent_prep : RMS-norm of the query latent, RMS-norm of c, rotation of k_rot, cache write
//   eia_latent_attn : rotation of q_rot, tiled online-softmax attention, sigmoid head gate
#include "eia_common.h"

// ------------------------------------------------------------------------------------------ prep
// fused [T, ld]: columns [q_off, q_off+q_rank) query latent, [c_off, c_off+R) KV latent,
// [kr_off, kr_off+rd) shared rotary key part.  q_rank == 0: no query latent; cache == nullptr:
// no KV part (a layer that reads another layer's cache).
template <typename T>
__global__ void __launch_bounds__(128)
latent_prep_kernel(const T* __restrict__ fused, long ld, int q_off, int q_rank,
                   const T* __restrict__ wq, T* __restrict__ cq, long ldcq, int c_off, int R,
                   const T* __restrict__ wc, int kr_off, int rd, int rot_dims,
                   const float* __restrict__ inv_freq, const int* __restrict__ positions,
                   const int* __restrict__ slot_mapping, T* __restrict__ cache, long cache_row,
                   float eps) {
  __shared__ float scratch[2];
  const long t = blockIdx.x;
  const T* row = fused + t * ld;
  if (q_rank > 0) {
    float ss = 0.f;
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x) {
      const float v = ld_f32<T>(row, q_off + c);
      ss += v * v;
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)q_rank + eps);
    for (int c = threadIdx.x; c < q_rank; c += blockDim.x)
      st_f32<T>(cq + t * ldcq, c, ld_f32<T>(row, q_off + c) * inv * ld_f32<T>(wq, c));
  }
  if (cache == nullptr) return;
  const int slot = slot_mapping[t];
  if (slot < 0) return;                       // uniform per workgroup
  T* dst = cache + (long)slot * cache_row;
  float ss = 0.f;
  for (int c = threadIdx.x; c < R; c += blockDim.x) {
    const float v = ld_f32<T>(row, c_off + c);
    ss += v * v;
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)R + eps);
  for (int c = threadIdx.x; c < R; c += blockDim.x)
    st_f32<T>(dst, c, ld_f32<T>(row, c_off + c) * inv * ld_f32<T>(wc, c));
  const float pos = (float)positions[t];
  for (int d = threadIdx.x; d < rd; d += blockDim.x) {
    float v = ld_f32<T>(row, kr_off + d);
    if (d < rot_dims) {
      const int i = d >> 1;
      float sn, cs;
      sincosf(pos * inv_freq[i], &sn, &cs);
      const float u = ld_f32<T>(row, kr_off + 2 * i), w = ld_f32<T>(row, kr_off + 2 * i + 1);
      v = (d & 1) ? (w * cs + u * sn) : (u * cs - w * sn);
    }
    st_f32<T>(dst, R + d, v);
  }
}

EIA_API int eia_latent_prep(const void* fused, long ld, int q_off, int q_rank, const void* wq,
                            void* cq, long ldcq, int c_off, int R, const void* wc, int kr_off,
                            int rd, int rot_dims, const float* inv_freq, const int* positions,
                            const int* slot_mapping, void* cache, long cache_row, float eps,
                            int T_, int is_bf16, hipStream_t st) {
  if (T_ < 0 || q_rank < 0 || (cache && (R < 1 || rd < 0 || rot_dims > rd || (rot_dims & 1))))
    return EIA_BAD_SHAPE;
  if (T_ == 0) return EIA_OK;
  if (is_bf16)
    hipLaunchKernelGGL((latent_prep_kernel<bf16_t>), dim3(T_), dim3(128), 0, st,
                       (const bf16_t*)fused, ld, q_off, q_rank, (const bf16_t*)wq, (bf16_t*)cq,
                       ldcq, c_off, R, (const bf16_t*)wc, kr_off, rd, rot_dims, inv_freq, positions,
                       slot_mapping, (bf16_t*)cache, cache_row, eps);
  else
    hipLaunchKernelGGL((latent_prep_kernel<float>), dim3(T_), dim3(128), 0, st,
                       (const float*)fused, ld, q_off, q_rank, (const float*)wq, (float*)cq, ldcq,
                       c_off, R, (const float*)wc, kr_off, rd, rot_dims, inv_freq, positions,
                       slot_mapping, (float*)cache, cache_row, eps);
  EIA_LAUNCH_CHECK();
}

// ------------------------------------------------------------------------------------- attention
#define LAT_ACC_MAX 32     // fp32 accumulators per thread: QB * HB * R <= 256 * LAT_ACC_MAX

struct LatentAttnArgs {
  const void* qa; long qa_st, qa_sh;        // absorbed queries (t, h, r)
  const void* qr; long qr_st, qr_sh;        // rotary query part, not yet rotated (t, h, d)
  const float* inv_freq; int rot_dims;
  const void* cache; long cache_row;        // rows of R + rd
  const int* block_table; int bt_stride;
  const int* seq_lens;                      // nullable: rows with 0 are padding
  const int* cu_q;                          // nullable: one query per sequence (decode)
  const int* work; int n_work;              // nullable with cu_q == nullptr: item = sequence
  const int* positions;                     // per query row
  const void* gate; long gate_st;           // nullable: sigmoid(gate[t][h]) scales head h
  void* out; long out_st, out_sh;           // (t, h, r)
  float scale; int H, R, rd, bs, QB, HB, KC, ldk;
};

template <typename T>
__global__ void __launch_bounds__(256)
latent_attn_kernel(LatentAttnArgs a) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int Dk = a.R + a.rd, M = a.QB * a.HB, KC = a.KC, ldk = a.ldk;
  float* qs = reinterpret_cast<float*>(smem);            // [M][Dk]
  float* ps = qs + (long)M * Dk;                         // [M][KC]
  float* mrow = ps + (long)M * KC;                       // [M]
  float* lrow = mrow + M;                                // [M]
  float* arow = lrow + M;                                // [M]
  T* kt = reinterpret_cast<T*>(arow + M);                // [KC][ldk]

  int seq, row0, ntok;
  if (a.cu_q) {
    seq = a.work[2 * blockIdx.x];
    const int q0 = a.work[2 * blockIdx.x + 1];
    const int lo = a.cu_q[seq], hi = a.cu_q[seq + 1];
    row0 = lo + q0;
    ntok = min(a.QB, hi - row0);
  } else {
    seq = blockIdx.x;
    row0 = seq;
    ntok = 1;
  }
  if (ntok <= 0 || (a.seq_lens && a.seq_lens[seq] <= 0)) return;
  const int h0 = blockIdx.y * a.HB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* qa = static_cast<const T*>(a.qa);
  const T* qr = static_cast<const T*>(a.qr);
  const T* cache = static_cast<const T*>(a.cache);
  const int* bt = a.block_table + (long)seq * a.bt_stride;

  // queries -> LDS (rotated, pre-scaled); rows of absent tokens / heads are zero
  for (int e = tid; e < M * Dk; e += 256) {
    const int m = e / Dk, d = e - m * Dk;
    const int t = m / a.HB, h = h0 + (m - t * a.HB);
    float v = 0.f;
    if (t < ntok && h < a.H) {
      const long row = row0 + t;
      if (d < a.R) {
        v = ld_f32<T>(qa, row * a.qa_st + h * a.qa_sh + d);
      } else {
        const int dd = d - a.R;
        const T* src = qr + row * a.qr_st + h * a.qr_sh;
        v = ld_f32<T>(src, dd);
        if (dd < a.rot_dims) {
          const int i = dd >> 1;
          float sn, cs;
          sincosf((float)a.positions[row] * a.inv_freq[i], &sn, &cs);
          const float u = ld_f32<T>(src, 2 * i), w = ld_f32<T>(src, 2 * i + 1);
          v = (dd & 1) ? (w * cs + u * sn) : (u * cs - w * sn);
        }
      }
      v *= a.scale;
    }
    qs[e] = v;
  }
  for (int m = tid; m < M; m += 256) {
    mrow[m] = -INFINITY;
    lrow[m] = 0.f;
    arow[m] = 1.f;
  }
  float acc[LAT_ACC_MAX];
#pragma unroll
  for (int i = 0; i < LAT_ACC_MAX; ++i) acc[i] = 0.f;
  const int nacc = (M * a.R + 255) >> 8;
  const int kmax = a.positions[row0 + ntok - 1] + 1;     // keys 0..kmax-1 are visible to the tile
  __syncthreads();

  for (int k0 = 0; k0 < kmax; k0 += KC) {
    // key tile -> LDS
    for (int e = tid; e < KC * Dk; e += 256) {
      const int j = e / Dk, d = e - j * Dk;
      const int kp = k0 + j;
      T v = (T)0.f;
      if (kp < kmax) {
        const long slot = (long)bt[kp / a.bs] * a.bs + (kp % a.bs);
        v = cache[slot * a.cache_row + d];
      }
      kt[j * ldk + d] = v;
    }
    __syncthreads();
    // scores: consecutive lanes take consecutive keys of one query row
    for (int e = tid; e < M * KC; e += 256) {
      const int m = e / KC, j = e - m * KC;
      const int t = m / a.HB;
      const int kp = k0 + j;
      float s = -INFINITY;
      if (t < ntok && kp <= a.positions[row0 + t]) {
        const float* q = qs + (long)m * Dk;
        const T* k = kt + (long)j * ldk;
        s = 0.f;
        for (int d = 0; d < Dk; ++d) s += q[d] * ld_f32<T>(k, d);
      }
      ps[e] = s;
    }
    __syncthreads();
    // online softmax per row: one wave per row, lanes over the tile's keys
    for (int m = wave; m < M; m += 4) {
      float tmax = -INFINITY;
      for (int j = lane; j < KC; j += 64) tmax = fmaxf(tmax, ps[m * KC + j]);
      tmax = wave_max(tmax);
      const float mold = mrow[m];
      const float mnew = fmaxf(mold, tmax);
      float psum = 0.f;
      for (int j = lane; j < KC; j += 64) {
        const float s = ps[m * KC + j];
        const float p = (s == -INFINITY) ? 0.f : expf(s - mnew);
        ps[m * KC + j] = p;
        psum += p;
      }
      psum = wave_sum(psum);
      if (lane == 0) {
        const float al = (mold == -INFINITY) ? ((mnew == -INFINITY) ? 1.f : 0.f) : expf(mold - mnew);
        arow[m] = al;
        lrow[m] = lrow[m] * al + psum;
        mrow[m] = mnew;
      }
    }
    __syncthreads();
    // accumulate the latent part of the keys
#pragma unroll
    for (int i = 0; i < LAT_ACC_MAX; ++i) {
      if (i < nacc) {
        const int e = tid + (i << 8);
        const int m = e / a.R, r = e - m * a.R;
        if (m < M) {
          float v = acc[i] * arow[m];
          const float* p = ps + (long)m * KC;
          for (int j = 0; j < KC; ++j) v += p[j] * ld_f32<T>(kt, (long)j * ldk + r);
          acc[i] = v;
        }
      }
    }
    __syncthreads();
  }

  T* out = static_cast<T*>(a.out);
  const T* gate = static_cast<const T*>(a.gate);
#pragma unroll
  for (int i = 0; i < LAT_ACC_MAX; ++i) {
    if (i < nacc) {
      const int e = tid + (i << 8);
      const int m = e / a.R, r = e - m * a.R;
      if (m < M) {
        const int t = m / a.HB, h = h0 + (m - t * a.HB);
        if (t < ntok && h < a.H) {
          const long row = row0 + t;
          float v = acc[i] / lrow[m];
          if (gate) v *= 1.0f / (1.0f + expf(-ld_f32<T>(gate, row * a.gate_st + h)));
          st_f32<T>(out, row * a.out_st + h * a.out_sh + r, v);
        }
      }
    }
  }
}

// n_items: sequences (cu_q == nullptr, one query row per sequence) or work items (seq, first
// query) of QB queries each.  Heads are processed HB at a time (grid.y).
EIA_API int eia_latent_attn(const void* qa, long qa_st, long qa_sh, const void* qr, long qr_st,
                            long qr_sh, const float* inv_freq, int rot_dims, const void* cache,
                            long cache_row, const int* block_table, int bt_stride,
                            const int* seq_lens, const int* cu_q, const int* work, int n_items,
                            const int* positions, const void* gate, long gate_st, void* out,
                            long out_st, long out_sh, float scale, int H, int R, int rd, int bs,
                            int QB, int is_bf16, hipStream_t st) {
  if (H < 1 || R < 1 || rd < 0 || bs < 1 || QB < 1 || rot_dims > rd || (rot_dims & 1) ||
      cache_row < R + rd || (cu_q && !work))
    return EIA_BAD_SHAPE;
  if (n_items <= 0) return EIA_OK;
  int HB = H < 16 ? H : 16;
  while (HB > 1 && (long)QB * HB * R > 256L * LAT_ACC_MAX) HB = (HB + 1) / 2;
  if ((long)QB * HB * R > 256L * LAT_ACC_MAX) return EIA_UNSUPPORTED;
  const int Dk = R + rd, M = QB * HB;
  const int esz = is_bf16 ? 2 : 4;
  // key-tile row stride: an odd number of 32-bit words, so lanes reading one column of
  // consecutive rows hit distinct LDS banks
  int ldk = Dk;
  if (is_bf16) { ldk += ldk & 1; if (((ldk / 2) & 1) == 0) ldk += 2; }
  else if ((ldk & 1) == 0) ldk += 1;
  int KC = 64;
  size_t lds = 0;
  for (;; KC >>= 1) {
    lds = ((size_t)M * Dk + (size_t)M * KC + 3 * (size_t)M) * 4 + (size_t)KC * ldk * esz;
    if (lds <= 96 * 1024 || KC == 8) break;
  }
  if (lds > 150 * 1024) return EIA_UNSUPPORTED;
  LatentAttnArgs a{qa, qa_st, qa_sh, qr, qr_st, qr_sh, inv_freq, rot_dims, cache, cache_row,
                   block_table, bt_stride, seq_lens, cu_q, work, n_items, positions, gate, gate_st,
                   out, out_st, out_sh, scale, H, R, rd, bs, QB, HB, KC, ldk};
  dim3 grid(n_items, (H + HB - 1) / HB);
  if (is_bf16) {
    if (lds > 48 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_kernel<bf16_t>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((latent_attn_kernel<bf16_t>), grid, dim3(256), lds, st, a);
  } else {
    if (lds > 48 * 1024)
      (void)hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_kernel<float>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL((latent_attn_kernel<float>), grid, dim3(256), lds, st, a);
  }
  EIA_LAUNCH_CHECK();
}
