// Linear-attention recurrence with per-channel data-dependent decay (RWKV-style "wkv" mixing)
// on per-sequence state slots.
//
// State of a sequence and layer: S [heads, dk, dv] fp32 and the previous token's layer input
// prev [width] fp32.  A sequence whose first scheduled position is 0 starts from zeros whatever
// its slot held before, so slots are reused without clearing.
//
//   eia_token_shift_mix : mix_s[t] = x[t] + (x[t-1] - x[t]) * mu_s  for NS streams (x[-1] from
//                         the slot; zeros at position 0)
//   eia_wkv_scan        : w = exp(-exp(dec + w0));  o = (S + diag(u) k v^T)^T r;
//                         S = diag(w) S + k v^T;  y = o / rms(o) * norm_w * silu(g)
//                         and prev <- x[last token of the step]
//
// Batch layout: sequence s owns rows [cu[s], cu[s+1]) (cu == nullptr: row s).  All recurrence
// math is fp32; activations are bf16 or fp32 (template T).
#include "eia_common.h"

EIA_DEV int find_seq(const int* cu, int nseq, int row) {
  int lo = 0, hi = nseq - 1;               // largest s with cu[s] <= row
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (cu[mid] <= row) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_mix_kernel(const float* __restrict__ x, const T* __restrict__ mu, int NS,
                       const float* __restrict__ prev_state, const int* __restrict__ slots,
                       const int* __restrict__ cu, int nseq, const int* __restrict__ positions,
                       T* __restrict__ out, long out_ss, int W) {
  const int row = blockIdx.x;
  const int s = cu ? find_seq(cu, nseq, row) : row;
  const int first = cu ? cu[s] : row;
  const float* cur = x + (long)row * W;
  const float* prv = nullptr;
  if (row > first) prv = cur - W;
  else if (positions[row] > 0 && slots[s] >= 0) prv = prev_state + (long)slots[s] * W;
  for (int c = threadIdx.x; c < W; c += blockDim.x) {
    const float a = cur[c];
    const float d = (prv ? prv[c] : 0.f) - a;
    for (int k = 0; k < NS; ++k)
      st_f32<T>(out + (long)k * out_ss + (long)row * W, c, a + d * ld_f32<T>(mu, (long)k * W + c));
  }
}

// x fp32 [rows, W]; mu [NS, W]; out [NS, rows, W] (stream stride out_ss elements).
EIA_API int eia_token_shift_mix(const float* x, const void* mu, int NS, const float* prev_state,
                                const int* slots, const int* cu, int nseq, const int* positions,
                                void* out, long out_ss, int rows, int W, int is_bf16,
                                hipStream_t st) {
  if (rows < 0 || W < 1 || NS < 1 || nseq < 1) return EIA_BAD_SHAPE;
  if (rows == 0) return EIA_OK;
  if (is_bf16)
    hipLaunchKernelGGL((token_shift_mix_kernel<bf16_t>), dim3(rows), dim3(256), 0, st, x,
                       (const bf16_t*)mu, NS, prev_state, slots, cu, nseq, positions,
                       (bf16_t*)out, out_ss, W);
  else
    hipLaunchKernelGGL((token_shift_mix_kernel<float>), dim3(rows), dim3(256), 0, st, x,
                       (const float*)mu, NS, prev_state, slots, cu, nseq, positions, (float*)out,
                       out_ss, W);
  EIA_LAUNCH_CHECK();
}

struct WkvArgs {
  const void *r, *k, *v, *g; long ld;       // [rows, H*D] each, row stride ld
  const float* dec; long ld_dec;            // [rows, H*D] fp32 decay pre-activation (without w0)
  const void *w0, *u, *norm_w;              // [H*D] each
  float* S;                                 // [slots, H, D, D]
  float* prev; const float* x; int W;       // prev [slots, W]; x fp32 [rows, W]
  const int* slots; const int* cu; const int* positions; const int* seq_lens;
  void* y; long ldy;                        // [rows, H*D]
  float eps; int H, D;
};

// One workgroup per (sequence, head), 4 x max(64, DMAX) threads: thread (q, j) owns rows
// [q DMAX/4, (q+1) DMAX/4) of column j of S in registers and walks the sequence's tokens in
// order.  Tokens are staged TC at a time: r, k, decay, v and the gate of TC tokens go to LDS
// (coalesced over the channels; channels >= D hold zeros so the dk loops run branch-free), the
// recurrence runs TC steps on LDS broadcasts leaving four partial outputs per token and column,
// and the partials are then summed, RMS-normed per head, weighted and gated -- so a token costs
// a quarter pass over dk per thread instead of a global-memory round trip.
template <typename T, int DMAX>
__global__ void __launch_bounds__(4 * (DMAX < 64 ? 64 : DMAX))
wkv_scan_kernel(WkvArgs a) {
  constexpr int DP = DMAX < 64 ? 64 : DMAX;          // threads per quarter
  constexpr int DQ = DMAX / 4;                       // dk rows per thread
  constexpr int TC = DMAX <= 64 ? 16 : DMAX <= 128 ? 8 : 4;
  constexpr int NWV = DP / 64;                       // waves per quarter
  __shared__ __align__(16) float sr[TC][DMAX], sk[TC][DMAX], sw[TC][DMAX], su[DMAX];
  __shared__ float sv[TC][DMAX], sg[TC][DMAX], po[TC][4][DP];
  __shared__ float red[4][NWV];
  const int s = blockIdx.x, h = blockIdx.y, D = a.D;
  const int q = threadIdx.x / DP, j = threadIdx.x % DP;
  const int slot = a.slots[s];
  if (slot < 0 || (a.seq_lens && a.seq_lens[s] <= 0)) return;
  const int lo = a.cu ? a.cu[s] : s, hi = a.cu ? a.cu[s + 1] : s + 1;
  if (hi <= lo) return;
  const bool fresh = a.positions[lo] == 0;
  const bool live = j < D, mine = j < DMAX;
  float* Sg = a.S + ((long)slot * a.H + h) * D * D;
  const int i0 = q * DQ;
  float S[DQ];
#pragma unroll
  for (int i = 0; i < DQ; ++i)
    S[i] = (!fresh && i0 + i < D && live) ? Sg[(long)(i0 + i) * D + j] : 0.f;
  const long hc = (long)h * D;
  if (q == 0 && mine) su[j] = live ? ld_f32<T>(static_cast<const T*>(a.u), hc + j) : 0.f;
  const float w0 = live ? ld_f32<T>(static_cast<const T*>(a.w0), hc + j) : 0.f;
  const float nw = live ? ld_f32<T>(static_cast<const T*>(a.norm_w), hc + j) : 0.f;
  const T* R = static_cast<const T*>(a.r);
  const T* K = static_cast<const T*>(a.k);
  const T* V = static_cast<const T*>(a.v);
  const T* G = static_cast<const T*>(a.g);
  T* Y = static_cast<T*>(a.y);
  const float inv_d = 1.0f / (float)D;
  for (int base = lo; base < hi; base += TC) {
    const int nt = min(TC, hi - base);
    __syncthreads();                       // the previous chunk's LDS reads are done
    if (mine) {
#pragma unroll
      for (int tt = 0; tt < TC / 4; ++tt) {            // quarter q stages tokens q, q + 4, ...
        const int t = tt * 4 + q;
        if (t < nt) {
          const long row = base + t;
          float r = 0.f, k = 0.f, w = 0.f, v = 0.f, g = 0.f;
          if (live) {
            r = ld_f32<T>(R, row * a.ld + hc + j);
            k = ld_f32<T>(K, row * a.ld + hc + j);
            w = expf(-expf(a.dec[row * a.ld_dec + hc + j] + w0));
            v = ld_f32<T>(V, row * a.ld + hc + j);
            g = ld_f32<T>(G, row * a.ld + hc + j);
          }
          sr[t][j] = r;
          sk[t][j] = k;
          sw[t][j] = w;
          sv[t][j] = v;
          sg[t][j] = g;
        }
      }
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float v = mine ? sv[t][j] : 0.f;
      float o = 0.f;
#pragma unroll
      for (int i = 0; i < DQ; ++i) {
        const float kv = sk[t][i0 + i] * v;
        o += sr[t][i0 + i] * (S[i] + su[i0 + i] * kv);
        S[i] = sw[t][i0 + i] * S[i] + kv;
      }
      po[t][q][j] = o;
    }
    __syncthreads();
    // quarter q finishes tokens q, q + 4, ...: sum of the partials, head RMS norm, weight, gate
#pragma unroll
    for (int tt = 0; tt < TC / 4; ++tt) {
      const int t = tt * 4 + q;
      const bool ok = t < nt && live;
      const float o = ok ? po[t][0][j] + po[t][1][j] + po[t][2][j] + po[t][3][j] : 0.f;
      float ss = wave_sum(o * o);
      if (NWV > 1) {
        __syncthreads();
        if ((j & 63) == 0) red[q][j >> 6] = ss;
        __syncthreads();
        ss = 0.f;
#pragma unroll
        for (int x = 0; x < NWV; ++x) ss += red[q][x];
      }
      if (ok) {
        const float g = sg[t][j];
        const float gate = g / (1.0f + expf(-g));
        st_f32<T>(Y, (long)(base + t) * a.ldy + hc + j, o / sqrtf(ss * inv_d + a.eps) * nw * gate);
      }
    }
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DQ; ++i)
      if (i0 + i < D) Sg[(long)(i0 + i) * D + j] = S[i];
  }
  if (h == 0) {
    const float* last = a.x + (long)(hi - 1) * a.W;
    float* p = a.prev + (long)slot * a.W;
    for (int c = threadIdx.x; c < a.W; c += blockDim.x) p[c] = last[c];
  }
}

EIA_API int eia_wkv_scan(const void* r, const void* k, const void* v, const void* g, long ld,
                         const float* dec, long ld_dec, const void* w0, const void* u,
                         const void* norm_w, float* S, float* prev, const float* x, int W,
                         const int* slots, const int* cu, const int* positions,
                         const int* seq_lens, void* y, long ldy, float eps, int nseq, int H, int D,
                         int is_bf16, hipStream_t st) {
  if (nseq < 0 || H < 1 || D < 1 || W < 1) return EIA_BAD_SHAPE;
  if (D > 256) return EIA_UNSUPPORTED;
  if (nseq == 0) return EIA_OK;
  WkvArgs a{r, k, v, g, ld, dec, ld_dec, w0, u, norm_w, S, prev, x, W, slots, cu, positions,
            seq_lens, y, ldy, eps, H, D};
  dim3 grid(nseq, H);
#define WKV_LAUNCH(TT, DM)                                                                 \
  hipLaunchKernelGGL((wkv_scan_kernel<TT, DM>), grid, dim3(4 * (DM < 64 ? 64 : DM)), 0, st, a)
  if (is_bf16) {
    if (D <= 32) WKV_LAUNCH(bf16_t, 32);
    else if (D <= 64) WKV_LAUNCH(bf16_t, 64);
    else if (D <= 128) WKV_LAUNCH(bf16_t, 128);
    else WKV_LAUNCH(bf16_t, 256);
  } else {
    if (D <= 32) WKV_LAUNCH(float, 32);
    else if (D <= 64) WKV_LAUNCH(float, 64);
    else if (D <= 128) WKV_LAUNCH(float, 128);
    else WKV_LAUNCH(float, 256);
  }
#undef WKV_LAUNCH
  EIA_LAUNCH_CHECK();
}
