// Sliding-window attention over a paged key / value cache with
//   * a logarithmic distance bias:   s = scale q.k - r1[h] ln(1 + r2[h] (i - j)),
//   * a sink in the softmax:         p_j = exp(s_j) / (1 + sum_j exp(s_j))  (a key of score 0, no value),
//   * mixing of the heads' weights:  w_h(i, j) = sum_g talk[h][g] p_g(i, j),
// and grouped key / value heads (query head h reads head h / (H / G)).  Position i sees
// j with 0 <= i - j < window.
//
// Pages: kc [pages][BS][G * D], vc [pages][BS][G * V], a token's slot = page * BS + offset.
// The query rows come from the joint projection (q | k | v) with row stride qs.
// Scores, weights and accumulation are fp32; TA (bf16 as uint16_t, or float) is the type of
// q, the pages and the output.
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldw(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldw<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldw<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void stw(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void stw<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void stw<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

// The k and v parts of the joint projection's rows go to their pages.
template <typename TA>
__global__ void __launch_bounds__(256) window_kv_write_kernel(const TA* __restrict__ qkv, int qs, int k_off, int nk,
                                                              int nv, const int* __restrict__ slots,
                                                              TA* __restrict__ kc, TA* __restrict__ vc) {
  const int t = blockIdx.x, sl = slots[t];
  if (sl < 0) return;
  const TA* row = qkv + (size_t)t * qs + k_off;
  for (int c = threadIdx.x; c < nk; c += 256) kc[(size_t)sl * nk + c] = row[c];
  for (int c = threadIdx.x; c < nv; c += 256) vc[(size_t)sl * nv + c] = row[nk + c];
}

constexpr int kWinTile = 64;   // keys per tile: one per lane
constexpr int kWinOut = 16;    // outputs per thread: H * V <= 256 * kWinOut

// score of key j for head h of the row (q in LDS, fp32)
template <typename TA>
__device__ __forceinline__ float win_score(const float* q, const TA* __restrict__ kc, const int* __restrict__ bt,
                                           int BS, int NK, int D, int g, int j, int dist, float scale, float r1,
                                           float r2) {
  const TA* kr = kc + ((size_t)bt[j / BS] * BS + (j % BS)) * NK + (size_t)g * D;
  float a = 0.f;
  for (int d = 0; d < D; ++d) a = fmaf(q[d], ldw(kr, d), a);
  return a * scale - r1 * log1pf(r2 * (float)dist);
}

// One workgroup per row, two passes over the window's keys in tiles of 64 (tile borders depend on
// the row's position only, so a row's result does not depend on the batch):
//   1. per head the maximum (the sink's 0 included) and the denominator, online;
//   2. scores again -> weights -> mixed over heads in LDS -> times the values.
template <typename TA>
__global__ void __launch_bounds__(256) window_attn_rows_kernel(const TA* __restrict__ qkv, int qs,
                                                               const TA* __restrict__ kc, const TA* __restrict__ vc,
                                                               const int* __restrict__ block_tables, int maxb,
                                                               const int* __restrict__ row_seg,
                                                               const int* __restrict__ seg_row0,
                                                               const int* __restrict__ seg_pos0,
                                                               const float* __restrict__ r1,
                                                               const float* __restrict__ r2,
                                                               const float* __restrict__ talk, TA* __restrict__ out,
                                                               int H, int G, int D, int V, int BS, int window,
                                                               float scale) {
  extern __shared__ float sm[];
  float* q = sm;                       // [H][D]
  float* p = q + H * D;                // [H][64]
  float* wm = p + H * kWinTile;        // [H][64]
  float* mh = wm + H * kWinTile;       // [H]
  float* lh = mh + H;                  // [H]
  float* tk = lh + H;                  // [H][H]
  const int r = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int sg = row_seg[r], pos = seg_pos0[sg] + r - seg_row0[sg];
  const int j_lo = max(0, pos - window + 1), j_hi = pos;
  const int* bt = block_tables + (size_t)sg * maxb;
  const int NK = G * D, NV = G * V, hpg = H / G;
  for (int i = tid; i < H * D; i += 256) q[i] = ldw(qkv, (size_t)r * qs + i);
  for (int i = tid; i < H * H; i += 256) tk[i] = talk[i];
  __syncthreads();
  for (int h = wv; h < H; h += 4) {
    const int g = h / hpg;
    const float a1 = r1[h], a2 = r2[h];
    float m = 0.f, l = 1.f;              // the sink: score 0, weight exp(0 - m)
    for (int j0 = j_lo; j0 <= j_hi; j0 += kWinTile) {
      const int j = j0 + lane;
      const bool ok = j <= j_hi;
      const float s = ok ? win_score(q + h * D, kc, bt, BS, NK, D, g, j, pos - j, scale, a1, a2) : -INFINITY;
      const float mn = fmaxf(m, wave_max(s));
      l = l * expf(m - mn) + wave_sum(ok ? expf(s - mn) : 0.f);
      m = mn;
    }
    if (lane == 0) {
      mh[h] = m;
      lh[h] = l;
    }
  }
  __syncthreads();
  float acc[kWinOut];
#pragma unroll
  for (int i = 0; i < kWinOut; ++i) acc[i] = 0.f;
  for (int j0 = j_lo; j0 <= j_hi; j0 += kWinTile) {
    for (int h = wv; h < H; h += 4) {
      const int j = j0 + lane;
      const bool ok = j <= j_hi;
      const float s = ok ? win_score(q + h * D, kc, bt, BS, NK, D, h / hpg, j, pos - j, scale, r1[h], r2[h]) : 0.f;
      p[h * kWinTile + lane] = ok ? expf(s - mh[h]) / lh[h] : 0.f;
    }
    __syncthreads();
    for (int i = tid; i < H * kWinTile; i += 256) {
      const int h = i / kWinTile, jj = i % kWinTile;
      float a = 0.f;
      for (int g = 0; g < H; ++g) a = fmaf(tk[h * H + g], p[g * kWinTile + jj], a);
      wm[i] = a;
    }
    __syncthreads();
    const int nk = min(kWinTile, j_hi - j0 + 1);
#pragma unroll
    for (int i = 0; i < kWinOut; ++i) {
      const int o = tid + i * 256;
      if (o < H * V) {
        const int h = o / V, v = o - h * V, g = h / hpg;
        float a = acc[i];
        for (int jj = 0; jj < nk; ++jj) {
          const int j = j0 + jj;
          a = fmaf(wm[h * kWinTile + jj], ldw(vc, ((size_t)bt[j / BS] * BS + (j % BS)) * NV + (size_t)g * V + v), a);
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < kWinOut; ++i) {
    const int o = tid + i * 256;
    if (o < H * V) stw(out, (size_t)r * H * V + o, acc[i]);
  }
}

}  // namespace k8s

using namespace k8s;

#define K8S_WDT(dt, ...)   \
  if ((dt) == 0) {          \
    using TA = uint16_t;    \
    __VA_ARGS__;            \
  } else {                  \
    using TA = float;       \
    __VA_ARGS__;            \
  }

K8S_API int k8s_window_kv_write(const void* qkv, int qs, int k_off, int nk, int nv, const int* slots, void* kc,
                                void* vc, int T, int dt, hipStream_t s) {
  if (T <= 0) return 0;
  K8S_WDT(dt, hipLaunchKernelGGL((window_kv_write_kernel<TA>), dim3(T), dim3(256), 0, s, (const TA*)qkv, qs, k_off, nk,
                                 nv, slots, (TA*)kc, (TA*)vc));
  return (int)hipGetLastError();
}

K8S_API int k8s_window_attn_rows(const void* qkv, int qs, const void* kc, const void* vc, const int* block_tables,
                                 int maxb, const int* row_seg, const int* seg_row0, const int* seg_pos0,
                                 const float* r1, const float* r2, const float* talk, void* out, int T, int H, int G,
                                 int D, int V, int BS, int window, float scale, int dt, hipStream_t s) {
  if (T <= 0) return 0;
  const size_t lds = (size_t)(H * D + 2 * H * kWinTile + 2 * H + H * H) * sizeof(float);
  if (H < 1 || G < 1 || H % G || H * V > 256 * kWinOut || window < 1 || lds > 64 * 1024)
    return (int)hipErrorInvalidValue;
  K8S_WDT(dt, hipLaunchKernelGGL((window_attn_rows_kernel<TA>), dim3(T), dim3(256), lds, s, (const TA*)qkv, qs,
                                 (const TA*)kc, (const TA*)vc, block_tables, maxb, row_seg, seg_row0, seg_pos0, r1,
                                 r2, talk, (TA*)out, H, G, D, V, BS, window, scale));
  return (int)hipGetLastError();
}
