// Windowed multi-map softmax attention over a paged, token-major K / V cache.
//
// A query row carries M = H * P score maps (H heads, P maps per head: 1 for ordinary heads, 2 for
// a differential pair), each D wide and already RMS-normed.  Map m = h * P + c of head h reads
// key map (h / (H / G)) * P + c of the token's key row ([G * P, D], normed at write time) and
// value head h / (H / G) of its value row ([G, Dv]).  For the pair (query position i, key j):
//
//   raw_m  = (q_m . k) * mult[m] - slope[m] * (i - j)            (slope == nullptr: no distance term)
//   s_h    = sum_g talk[h, g] * raw_g                             (talk == nullptr: s = raw)
//   visible: j <= i and (i - j < window or j < keep)              (window <= 0: every j <= i)
//   p      = softmax over the visible keys, per map;  a_m = sum_j p_mj v_j
//
// Epilogue 0: out[h] = a_h * sigmoid(gate[h])   (gate == nullptr: out = a; P must be 1)
// Epilogue 1: o = a_{2h} - lam * a_{2h+1};  out[h] = o / sqrt(mean(o^2) + eps) * post   (P == 2)
//
// Scores, softmax weights, accumulators, norms and gates are fp32 whatever the storage type.
// Rows are [decode rows (one per sequence) | prefill chunks]; both read the cache after
// qk_norm_cache wrote this step's tokens, so chunked prompts and mixed batches need no
// special path: a row is (position, block-table row) and nothing else.
#include "eia_common.h"

// ---------------------------------------------------------------------------------------------
// Cache write.  One workgroup per token of a fused projection row:
//   q maps  -> RMS norm (weight qw[D]) -> q_out[t, MQ * D]
//   k maps  -> RMS norm (weight kw[D]) -> key row of the token's slot
//   values  -> copied as projected     -> value row of the token's slot
// (values may alias the un-normed key columns: v_off == k_off).  Slots < 0 write no cache rows.
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_cache_kernel(const T* __restrict__ fused, long ld, int q_off, int k_off, int v_off,
                     int MQ, int MK, int D, int VW, const T* __restrict__ qw,
                     const T* __restrict__ kw, T* __restrict__ q_out, long ldq,
                     T* __restrict__ kc, T* __restrict__ vc, const int* __restrict__ slots,
                     float eps) {
  const long t = blockIdx.x;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  const T* row = fused + t * ld;
  const long slot = slots ? (long)slots[t] : -1;
  for (int u = wave; u < MQ + MK; u += nw) {
    const bool isq = u < MQ;
    const int m = isq ? u : u - MQ;
    if (!isq && slot < 0) continue;
    const T* src = row + (isq ? q_off : k_off) + m * D;
    float ss = 0.f;
    for (int d = lane; d < D; d += 64) {
      const float v = ld_f32<T>(src, d);
      ss += v * v;
    }
    const float inv = 1.0f / sqrtf(wave_sum(ss) / (float)D + eps);
    T* dst = isq ? q_out + t * ldq + m * D : kc + slot * ((long)MK * D) + m * D;
    const T* w = isq ? qw : kw;
    for (int d = lane; d < D; d += 64)
      st_f32<T>(dst, d, ld_f32<T>(src, d) * inv * ld_f32<T>(w, d));
  }
  if (slot >= 0) {
    const T* src = row + v_off;
    T* dst = vc + slot * (long)VW;
    for (int c = threadIdx.x; c < VW; c += blockDim.x) dst[c] = src[c];
  }
}

EIA_API int eia_qk_norm_cache(const void* fused, long ld, int q_off, int k_off, int v_off, int MQ,
                              int MK, int D, int VW, const void* qw, const void* kw, void* q_out,
                              long ldq, void* kc, void* vc, const int* slots, float eps, int T,
                              int is_bf16, hipStream_t st) {
  if (T < 0 || MQ < 1 || MK < 1 || D < 1 || VW < 1 || !fused || !q_out || !kc || !vc)
    return EIA_BAD_SHAPE;
  if (T == 0) return EIA_OK;
  if (is_bf16)
    hipLaunchKernelGGL((qk_norm_cache_kernel<bf16_t>), dim3(T), dim3(256), 0, st,
                       (const bf16_t*)fused, ld, q_off, k_off, v_off, MQ, MK, D, VW,
                       (const bf16_t*)qw, (const bf16_t*)kw, (bf16_t*)q_out, ldq, (bf16_t*)kc,
                       (bf16_t*)vc, slots, eps);
  else
    hipLaunchKernelGGL((qk_norm_cache_kernel<float>), dim3(T), dim3(256), 0, st,
                       (const float*)fused, ld, q_off, k_off, v_off, MQ, MK, D, VW,
                       (const float*)qw, (const float*)kw, (float*)q_out, ldq, (float*)kc,
                       (float*)vc, slots, eps);
  EIA_LAUNCH_CHECK();
}

// ---------------------------------------------------------------------------------------------
struct WinAttnArgs {
  const void* q; long ldq;          // [rows, M * D]
  const void* kc; const void* vc;   // [slots, G * P * D], [slots, G * Dv]
  const int* bt; int ldbt;          // block tables [seqs, ldbt]
  const int* positions;             // [rows]
  const int* cu;                    // prefill: first row of each sequence's chunk; decode: null
  const int* work;                  // prefill: (sequence, first query of the chunk) pairs
  const int* lens;                  // decode: sequence lengths (0: padding row)
  const float* mult;                // [M]
  const float* slope;               // [M] or null
  const float* talk;                // [M, M] or null
  const void* gate; long ldg;       // [rows, H * Dv] before the sigmoid, or null
  void* out; long ldo;              // [rows, H * Dv]
  int H, G, P, D, Dv, bs, window, keep, qb, epilogue;
  float lam, eps, post;
};

constexpr int WA_KT = 64;           // keys per tile = lanes of a wave
constexpr int WA_ACC = 16;          // (map, value column) accumulators per thread

// Scalar-FMA form (fp32 models; bf16 shapes the MFMA form does not take).  One workgroup of four
// waves per work item; its queries run one after the other.  Per 64-key tile: (1) lane = key,
// the waves split the maps: raw scores into LDS; (2) the waves split the mixed maps: head mixing,
// mask, running max / sum with wave reductions, weights into LDS; (3) threads split the (map,
// value column) outputs and sweep the tile.
template <typename T>
__global__ void __launch_bounds__(256)
window_attn_kernel(const WinAttnArgs a) {
  extern __shared__ float lds[];
  const int H = a.H, P = a.P, D = a.D, Dv = a.Dv, M = H * P, rep = H / a.G;
  float* qs = lds;                        // [M, D]
  float* sraw = qs + M * D;               // [M, 64]
  float* pw = sraw + M * WA_KT;           // [M, 64]
  float* fin = pw + M * WA_KT;            // [M, Dv]
  float* mrun = fin + M * Dv;             // [M]
  float* lrun = mrun + M;                 // [M]
  float* alpha = lrun + M;                // [M]
  long* kslot = reinterpret_cast<long*>(alpha + M + (M & 1));   // [64], 8-byte aligned
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const T* q = (const T*)a.q;
  const T* kc = (const T*)a.kc;
  const T* vc = (const T*)a.vc;
  const T* gate = (const T*)a.gate;
  T* out = (T*)a.out;
  const long krow = (long)a.G * P * D, vrow = (long)a.G * Dv;

  int seq, row0, nq;
  if (a.cu) {
    seq = a.work[2 * blockIdx.x];
    const int q0 = a.work[2 * blockIdx.x + 1];
    const int n = a.cu[seq + 1] - a.cu[seq];
    row0 = a.cu[seq] + q0;
    nq = min(a.qb, n - q0);
  } else {
    seq = blockIdx.x;
    row0 = seq;
    nq = 1;
  }
  const int* bt = a.bt + (long)seq * a.ldbt;
  const int outw = H * Dv;

  for (int qi = 0; qi < nq; ++qi) {
    const long row = row0 + qi;
    if (a.lens && a.lens[seq] <= 0) {                  // padding row of a fixed-size batch
      for (int c = tid; c < outw; c += 256) st_f32<T>(out + row * a.ldo, c, 0.f);
      continue;
    }
    const int pos = a.positions[row];
    const int lo = a.window > 0 ? max(0, pos - a.window + 1) : 0;
    const int nsink = min(a.keep, lo);
    const int nkeys = nsink + pos - lo + 1;
    __syncthreads();                                   // previous query's LDS reads are over
    for (int c = tid; c < M * D; c += 256) qs[c] = ld_f32<T>(q + row * a.ldq, c);
    for (int m = tid; m < M; m += 256) { mrun[m] = -INFINITY; lrun[m] = 0.f; }
    float acc[WA_ACC];
#pragma unroll
    for (int i = 0; i < WA_ACC; ++i) acc[i] = 0.f;

    for (int k0 = 0; k0 < nkeys; k0 += WA_KT) {
      const int kk = k0 + lane;
      const bool valid = kk < nkeys;
      const int j = valid ? (kk < nsink ? kk : lo + kk - nsink) : pos;
      const long slot = (long)bt[j / a.bs] * a.bs + j % a.bs;
      __syncthreads();                                 // qs / mrun ready; last tile's reads over
      if (wave == 0) kslot[lane] = slot;
      // (1) raw scores of this lane's key
      for (int m = wave; m < M; m += 4) {
        const int h = m / P, c = m - h * P;
        const T* kp = kc + slot * krow + ((h / rep) * P + c) * D;
        const float* qp = qs + m * D;
        float s = 0.f;
        for (int d = 0; d < D; ++d) s += qp[d] * ld_f32<T>(kp, d);
        s *= a.mult[m];
        if (a.slope) s -= a.slope[m] * (float)(pos - j);
        sraw[m * WA_KT + lane] = s;
      }
      __syncthreads();
      // (2) head mixing, mask, online softmax
      for (int m = wave; m < M; m += 4) {
        float s;
        if (a.talk) {
          s = 0.f;
          for (int g = 0; g < M; ++g) s += a.talk[m * M + g] * sraw[g * WA_KT + lane];
        } else {
          s = sraw[m * WA_KT + lane];
        }
        if (!valid) s = -INFINITY;
        const float mo = mrun[m];
        const float mn = fmaxf(mo, wave_max(s));
        const float p = valid ? expf(s - mn) : 0.f;
        const float ps = wave_sum(p);
        pw[m * WA_KT + lane] = p;
        if (lane == 0) {
          const float al = expf(mo - mn);              // exp(-inf) = 0 at the first tile
          alpha[m] = al;
          lrun[m] = lrun[m] * al + ps;
          mrun[m] = mn;
        }
      }
      __syncthreads();
      // (3) weighted values
      const int nk = min(WA_KT, nkeys - k0);
#pragma unroll
      for (int i = 0; i < WA_ACC; ++i) {
        const int idx = tid + i * 256;
        if (idx < M * Dv) {
          const int m = idx / Dv, d = idx - m * Dv;
          const T* vp = vc + ((m / P) / rep) * Dv + d;
          const float* pm = pw + m * WA_KT;
          float s = acc[i] * alpha[m];
          for (int k = 0; k < nk; ++k) s += pm[k] * ld_f32<T>(vp, kslot[k] * vrow);
          acc[i] = s;
        }
      }
    }
    __syncthreads();
    if (a.epilogue == 0) {
#pragma unroll
      for (int i = 0; i < WA_ACC; ++i) {
        const int idx = tid + i * 256;
        if (idx < M * Dv) {
          float v = acc[i] / lrun[idx / Dv];
          if (gate) v *= 1.0f / (1.0f + expf(-ld_f32<T>(gate + row * a.ldg, idx)));
          st_f32<T>(out + row * a.ldo, idx, v);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < WA_ACC; ++i) {
        const int idx = tid + i * 256;
        if (idx < M * Dv) fin[idx] = acc[i] / lrun[idx / Dv];
      }
      __syncthreads();
      for (int h = wave; h < H; h += 4) {
        const float* a1 = fin + (2 * h) * Dv;
        const float* a2 = a1 + Dv;
        float ss = 0.f;
        for (int d = lane; d < Dv; d += 64) {
          const float o = a1[d] - a.lam * a2[d];
          ss += o * o;
        }
        const float inv = a.post / sqrtf(wave_sum(ss) / (float)Dv + a.eps);
        for (int d = lane; d < Dv; d += 64)
          st_f32<T>(out + row * a.ldo, h * Dv + d, (a1[d] - a.lam * a2[d]) * inv);
      }
    }
  }
}

static size_t wa_lds_bytes(int M, int D, int Dv) {
  return sizeof(float) * ((size_t)M * D + 2 * (size_t)M * WA_KT + (size_t)M * Dv + 3 * M + (M & 1))
         + sizeof(long) * WA_KT;
}

// n_items: decode rows (cu == nullptr) or prefill work items.
EIA_API int eia_window_attn(const void* q, long ldq, const void* kc, const void* vc, const int* bt,
                            int ldbt, const int* positions, const int* cu, const int* work,
                            const int* lens, int n_items, const float* mult, const float* slope,
                            const float* talk, const void* gate, long ldg, void* out, long ldo,
                            int H, int G, int P, int D, int Dv, int bs, int window, int keep,
                            int qb, int epilogue, float lam, float eps, float post, int is_bf16,
                            hipStream_t st) {
  if (n_items < 0 || H < 1 || G < 1 || H % G || (P != 1 && P != 2) || D < 1 || Dv < 1 || bs < 1 ||
      keep < 0 || qb < 1 || !q || !kc || !vc || !bt || !positions || !mult || !out)
    return EIA_BAD_SHAPE;
  if ((cu == nullptr) != (work == nullptr)) return EIA_BAD_SHAPE;
  if ((epilogue == 1) != (P == 2) || (epilogue == 1 && gate)) return EIA_BAD_SHAPE;
  const int M = H * P;
  const size_t lds = wa_lds_bytes(M, D, Dv);
  if (M * Dv > 256 * WA_ACC || lds > 64 * 1024) return EIA_UNSUPPORTED;
  if (n_items == 0) return EIA_OK;
  WinAttnArgs a{q, ldq, kc, vc, bt, ldbt, positions, cu, work, lens, mult, slope, talk, gate, ldg,
                out, ldo, H, G, P, D, Dv, bs, window, keep, qb, epilogue, lam, eps, post};
  if (is_bf16)
    hipLaunchKernelGGL((window_attn_kernel<bf16_t>), dim3(n_items), dim3(256), lds, st, a);
  else
    hipLaunchKernelGGL((window_attn_kernel<float>), dim3(n_items), dim3(256), lds, st, a);
  EIA_LAUNCH_CHECK();
}
