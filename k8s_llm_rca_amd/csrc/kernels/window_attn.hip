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

// The k and v parts of the joint projection's rows go to their pages; vt (optional) is the
// transposed twin of the value pages, [pages][G * V][BS]: the matrix-core kernel's PV operand.
template <typename TA>
__global__ void __launch_bounds__(256) window_kv_write_kernel(const TA* __restrict__ qkv, int qs, int k_off, int nk,
                                                              int nv, const int* __restrict__ slots,
                                                              TA* __restrict__ kc, TA* __restrict__ vc,
                                                              TA* __restrict__ vt, int BS) {
  const int t = blockIdx.x, sl = slots[t];
  if (sl < 0) return;
  const TA* row = qkv + (size_t)t * qs + k_off;
  for (int c = threadIdx.x; c < nk; c += 256) kc[(size_t)sl * nk + c] = row[c];
  for (int c = threadIdx.x; c < nv; c += 256) vc[(size_t)sl * nv + c] = row[nk + c];
  if (vt) {
    const int page = sl / BS, off = sl - page * BS;
    for (int c = threadIdx.x; c < nv; c += 256) vt[((size_t)page * nv + c) * BS + off] = row[nk + c];
  }
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


// ---------------------------------------------------------------------------------------------
// Matrix-core form (bf16, v_mfma_f32_16x16x32_bf16).  A workgroup of ceil(H / HW) waves owns a tile of up
// to 16 consecutive tokens of one segment; wave w owns the heads w HW .. w HW + HW - 1.  Keys go
// in blocks of 32 (never across a page: BS % 32 == 0).  Swapped QK^T as in the other attention
// kernels: a lane owns ONE query (lane & 15) and, per block, the scores of keys 8 q .. 8 q + 7 of its
// quarter q = lane >> 4 -- for every head at the same (query, key) positions, so mixing the heads'
// weights is element-wise across heads.
//   pass 1: per head and query the maximum (the sink's 0 included) and the denominator, online;
//   pass 2: scores again -> normalised weights of the wave's heads -> LDS -> every wave mixes all
//           heads' weights for its own heads (fp32) -> bf16 PV operand in place -> O += W V.
// The weights go through LDS double-buffered: one barrier per key block.
struct WinArgs {
  const uint16_t* qkv;    // [T][qs], the queries in the first H * D columns
  int qs;
  const uint16_t* kc;     // [pages][BS][G * D]
  const uint16_t* vt;     // [pages][G * V][BS]
  const int* bt;
  int maxb;
  const int* items;       // [n][4]: segment, first row, tokens (<= 16), position of the first token
  int n_items;
  const float* r1;
  const float* r2;
  const float* talk;
  uint16_t* out;          // [T][H * V]
  int H, G, BS, window;
  float scale;
  // split over the keys (steps of few rows): grid.y parts of part_keys keys (a multiple of 32) each
  int part_keys, n_parts;
  float* pml;             // [items][parts][H][16][2]: a part's maximum and denominator (log2 units)
  float* po;              // [items][parts][16][H * V]: a part's share of the output
};

__device__ __forceinline__ bf16x8 wld16(const uint16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
// 2^x on the hardware exponential; the arguments here are <= 0 or -inf (results in [0, 1], tiny ones flush to 0)
__device__ __forceinline__ float wexp2(float x) { return __builtin_amdgcn_exp2f(x); }

template <int NDC>
__device__ __forceinline__ void win_scores(const bf16x8 (&kf)[2][NDC], const bf16x8 (&qf)[NDC], int kb, int hq,
                                           int posq, bool qvalid, int window, float sl2, float c1, float c2,
                                           float (&p)[8]) {
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    f32x4 sacc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int cc = 0; cc < NDC; ++cc) sacc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][cc], qf[cc], sacc, 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int dist = posq - (kb + 8 * hq + 4 * t + i);
      const bool ok = qvalid && dist >= 0 && dist < window;
      // log2 units: scale q.k log2(e) - r1 log2(1 + r2 dist)
      p[4 * t + i] = ok ? sacc[i] * sl2 - c1 * __log2f(1.f + c2 * (float)dist) : -INFINITY;
    }
  }
}

// PHASE 0: both passes over all keys of the tile, bf16 output.  Split over the keys in three launches
// (part borders count from the tile's first key block: they depend on positions only):
// PHASE 1: pass 1 over one part, its (maximum, denominator) to pml;
// PHASE 2: all parts' pml merged, pass 2 over one part, its share of the output to po (fp32);
// window_attn_merge_kernel then adds the parts' shares.
template <int NDC, int NV, int HW, int PHASE>
__global__ void __launch_bounds__(512) window_attn_mfma_kernel(WinArgs a) {
  constexpr int D = NDC * 32, V = NV * 16;
  constexpr float kLog2e = 1.4426950408889634f;
  extern __shared__ float psm[];   // [2][H][2][64][4]: the normalised weights of one key block
  const int lane = threadIdx.x & 63, r = lane & 15, hq = lane >> 4;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int item = blockIdx.x;
  const int sg = a.items[item * 4], row0 = a.items[item * 4 + 1], ntok = a.items[item * 4 + 2],
            pos0 = a.items[item * 4 + 3];
  const int H = a.H, hpg = H / a.G, NK = a.G * D, NVt = a.G * V;
  const int h0 = wv * HW, nh = max(0, min(HW, H - h0));
  const int posq = pos0 + r;
  const bool qvalid = r < ntok;
  const int k_lo = max(0, pos0 - a.window + 1), k_hi = pos0 + ntok - 1;
  const float sl2 = a.scale * kLog2e;
  const int* pages = a.bt + (size_t)sg * a.maxb;
  const int part = PHASE ? blockIdx.y : 0;
  const int kb_first = (k_lo & ~31) + part * a.part_keys;
  const int kb_last = PHASE ? min(k_hi, kb_first + a.part_keys - 1) : k_hi;
  if (kb_first > k_hi) return;                     // an empty part (the whole workgroup leaves)
  bf16x8 qf[HW][NDC];
  float m2[HW], l[HW], c1[HW], c2[HW], inv_l[HW];
#pragma unroll
  for (int hh = 0; hh < HW; ++hh) {
    const bool on = hh < nh && qvalid;
    const uint16_t* qp = a.qkv + (size_t)(row0 + (on ? r : 0)) * a.qs + (size_t)(on ? h0 + hh : 0) * D;
#pragma unroll
    for (int cc = 0; cc < NDC; ++cc) {
      qf[hh][cc] = wld16(qp + 32 * cc + 8 * hq);
      if (!on)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[hh][cc][j] = (__bf16)0.f;
    }
    m2[hh] = 0.f;   // the sink's score
    l[hh] = 0.f;
    c1[hh] = hh < nh ? a.r1[h0 + hh] : 0.f;
    c2[hh] = hh < nh ? a.r2[h0 + hh] : 0.f;
  }
  // ---- pass 1: maximum and denominator
  if (PHASE != 2)
  for (int kb = kb_first; kb <= kb_last; kb += 32) {
    const int page = pages[kb / a.BS], off = kb % a.BS;
    const uint16_t* kp = a.kc + ((size_t)page * a.BS + off) * NK;
    bf16x8 kf[2][NDC];
    int gprev = -1;
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      if (hh < nh) {
        const int g = (h0 + hh) / hpg;
        if (g != gprev) {
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            const int key = 8 * (r >> 2) + 4 * t + (r & 3);
#pragma unroll
            for (int cc = 0; cc < NDC; ++cc) kf[t][cc] = wld16(kp + (size_t)key * NK + g * D + 32 * cc + 8 * hq);
          }
          gprev = g;
        }
        float p[8];
        win_scores<NDC>(kf, qf[hh], kb, hq, posq, qvalid, a.window, sl2, c1[hh], c2[hh], p);
        float cmax = p[0];
#pragma unroll
        for (int j = 1; j < 8; ++j) cmax = fmaxf(cmax, p[j]);
        cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
        cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
        const float mn = fmaxf(m2[hh], cmax);
        float ps = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) ps += wexp2(p[j] - mn);
        l[hh] = l[hh] * wexp2(m2[hh] - mn) + ps;
        m2[hh] = mn;
      }
    }
  }
#pragma unroll
  for (int hh = 0; hh < HW; ++hh) {
    if (PHASE != 2) {
      float lt = l[hh];
      lt += __shfl_xor(lt, 16, 64);
      lt += __shfl_xor(lt, 32, 64);
      l[hh] = lt;
    } else if (hh < nh) {                          // the parts' statistics, merged in part order
      float M = 0.f, L = 0.f;
      for (int p2 = 0; p2 < a.n_parts && (k_lo & ~31) + p2 * a.part_keys <= k_hi; ++p2) {
        const float* ml = a.pml + ((((size_t)item * a.n_parts + p2) * H + h0 + hh) * 16 + r) * 2;
        const float mp = ml[0], mn = fmaxf(M, mp);
        L = L * wexp2(M - mn) + ml[1] * wexp2(mp - mn);
        M = mn;
      }
      m2[hh] = M;
      l[hh] = L;
    }
    inv_l[hh] = 1.f / (l[hh] + wexp2(-m2[hh]));   // + the sink
  }
  if (PHASE == 1) {
    if (hq == 0)
#pragma unroll
      for (int hh = 0; hh < HW; ++hh)
        if (hh < nh) {
          float* ml = a.pml + ((((size_t)item * a.n_parts + part) * H + h0 + hh) * 16 + r) * 2;
          ml[0] = m2[hh];
          ml[1] = l[hh];
        }
    return;
  }
  // ---- pass 2: weights, mixed over heads, times the values
  f32x4 o[HW][NV];
#pragma unroll
  for (int hh = 0; hh < HW; ++hh)
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) o[hh][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  int buf = 0;
  for (int kb = kb_first; kb <= kb_last; kb += 32) {
    const int page = pages[kb / a.BS], off = kb % a.BS;
    const uint16_t* kp = a.kc + ((size_t)page * a.BS + off) * NK;
    float* P = psm + (size_t)buf * H * 512;
    {
      bf16x8 kf[2][NDC];
      int gprev = -1;
#pragma unroll
      for (int hh = 0; hh < HW; ++hh) {
        if (hh < nh) {
          const int g = (h0 + hh) / hpg;
          if (g != gprev) {
#pragma unroll
            for (int t = 0; t < 2; ++t) {
              const int key = 8 * (r >> 2) + 4 * t + (r & 3);
#pragma unroll
              for (int cc = 0; cc < NDC; ++cc) kf[t][cc] = wld16(kp + (size_t)key * NK + g * D + 32 * cc + 8 * hq);
            }
            gprev = g;
          }
          float p[8];
          win_scores<NDC>(kf, qf[hh], kb, hq, posq, qvalid, a.window, sl2, c1[hh], c2[hh], p);
          float* Ph = P + (size_t)(h0 + hh) * 512 + lane * 4;
#pragma unroll
          for (int t = 0; t < 2; ++t) {
            f32x4 e;
#pragma unroll
            for (int i = 0; i < 4; ++i) e[i] = wexp2(p[4 * t + i] - m2[hh]) * inv_l[hh];
            *reinterpret_cast<f32x4*>(Ph + t * 256) = e;
          }
        }
      }
    }
    __syncthreads();
    bf16x8 vf[NV];
    int gprev = -1;
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      if (hh < nh) {
        f32x4 w0 = f32x4{0.f, 0.f, 0.f, 0.f}, w1 = w0;
        const float* tk = a.talk + (size_t)(h0 + hh) * H;
        for (int g2 = 0; g2 < H; ++g2) {
          const float tv = tk[g2];
          const f32x4 e0 = *reinterpret_cast<const f32x4*>(P + (size_t)g2 * 512 + lane * 4);
          const f32x4 e1 = *reinterpret_cast<const f32x4*>(P + (size_t)g2 * 512 + 256 + lane * 4);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            w0[i] = fmaf(tv, e0[i], w0[i]);
            w1[i] = fmaf(tv, e1[i], w1[i]);
          }
        }
        bf16x8 pf;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          pf[i] = (__bf16)w0[i];
          pf[4 + i] = (__bf16)w1[i];
        }
        const int g = (h0 + hh) / hpg;
        if (g != gprev) {
          const uint16_t* vp = a.vt + ((size_t)page * NVt + (size_t)g * V) * a.BS + off + 8 * hq;
#pragma unroll
          for (int dt = 0; dt < NV; ++dt) vf[dt] = wld16(vp + (size_t)(16 * dt + r) * a.BS);
          gprev = g;
        }
#pragma unroll
        for (int dt = 0; dt < NV; ++dt) o[hh][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf, vf[dt], o[hh][dt], 0, 0, 0);
      }
    }
    buf ^= 1;
  }
#pragma unroll
  for (int hh = 0; hh < HW; ++hh) {
    if (hh < nh) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int q = 4 * hq + i;
        if (q < ntok) {
          if (PHASE == 2) {
            float* op = a.po + (((size_t)item * a.n_parts + part) * 16 + q) * H * V + (size_t)(h0 + hh) * V + r;
#pragma unroll
            for (int dt = 0; dt < NV; ++dt) op[16 * dt] = o[hh][dt][i];
          } else {
            uint16_t* op = a.out + (size_t)(row0 + q) * H * V + (size_t)(h0 + hh) * V + r;
#pragma unroll
            for (int dt = 0; dt < NV; ++dt) op[16 * dt] = f2bf(o[hh][dt][i]);
          }
        }
      }
    }
  }
}

// out = the sum of the parts' shares (in part order), one workgroup per tile
__global__ void __launch_bounds__(256) window_attn_merge_kernel(WinArgs a, int HV) {
  const int item = blockIdx.x;
  const int row0 = a.items[item * 4 + 1], ntok = a.items[item * 4 + 2], pos0 = a.items[item * 4 + 3];
  const int k_lo = max(0, pos0 - a.window + 1), k_hi = pos0 + ntok - 1;
  const int np = min(a.n_parts, (k_hi - (k_lo & ~31)) / a.part_keys + 1);
  for (int e = blockIdx.y * 256 + threadIdx.x; e < ntok * HV; e += gridDim.y * 256) {
    const int q = e / HV, c = e - q * HV;
    float acc = 0.f;
    for (int p2 = 0; p2 < np; ++p2) acc += a.po[(((size_t)item * a.n_parts + p2) * 16 + q) * HV + c];
    a.out[(size_t)(row0 + q) * HV + c] = f2bf(acc);
  }
}

template <int NDC, int NV, int HW, int PHASE>
static int launch_win_phase(const WinArgs& a, hipStream_t s) {
  const size_t lds = PHASE == 1 ? 0 : (size_t)2 * a.H * 512 * sizeof(float);
  auto k = window_attn_mfma_kernel<NDC, NV, HW, PHASE>;
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
    return (int)hipGetLastError();
  const int waves = (a.H + HW - 1) / HW;          // every wave owns HW heads (the last one maybe fewer)
  hipLaunchKernelGGL(k, dim3(a.n_items, PHASE ? a.n_parts : 1), dim3(64 * waves), lds, s, a);
  return (int)hipGetLastError();
}

template <int NDC, int NV, int HW>
static int launch_win_mfma(const WinArgs& a, hipStream_t s) {
  if (a.n_parts <= 1) return launch_win_phase<NDC, NV, HW, 0>(a, s);
  int rc = launch_win_phase<NDC, NV, HW, 1>(a, s);
  if (rc) return rc;
  rc = launch_win_phase<NDC, NV, HW, 2>(a, s);
  if (rc) return rc;
  hipLaunchKernelGGL(window_attn_merge_kernel, dim3(a.n_items, 16), dim3(256), 0, s, a, a.H * NV * 16);
  return (int)hipGetLastError();
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
                                void* vc, int T, int dt, hipStream_t s, void* vt, int BS) {
  if (T <= 0) return 0;
  if (vt && BS <= 0) return (int)hipErrorInvalidValue;
  K8S_WDT(dt, hipLaunchKernelGGL((window_kv_write_kernel<TA>), dim3(T), dim3(256), 0, s, (const TA*)qkv, qs, k_off, nk,
                                 nv, slots, (TA*)kc, (TA*)vc, (TA*)vt, BS));
  return (int)hipGetLastError();
}

// 1 when the matrix-core kernel takes these sizes (bf16 only)
K8S_API int k8s_window_attn_mfma_ok(int H, int G, int D, int V) {
  return H >= 1 && H <= 16 && G >= 1 && H % G == 0 && (D == 64 || D == 128) && (V == 64 || V == 128);
}

K8S_API int k8s_window_attn_mfma(const void* qkv, int qs, const void* kc, const void* vt, const int* block_tables,
                                 int maxb, const int* items, int n_items, const float* r1, const float* r2,
                                 const float* talk, void* out, int H, int G, int D, int V, int BS, int window,
                                 float scale, hipStream_t s, int part_keys, int n_parts, float* pml, float* po) {
  if (n_items <= 0) return 0;
  if (!k8s_window_attn_mfma_ok(H, G, D, V) || BS % 32 || window < 1 || qs % 8 || (D * G) % 8)
    return (int)hipErrorInvalidValue;
  if (n_parts > 1 && (part_keys < 32 || part_keys % 32 || !pml || !po)) return (int)hipErrorInvalidValue;
  WinArgs a;
  a.qkv = (const uint16_t*)qkv;
  a.qs = qs;
  a.kc = (const uint16_t*)kc;
  a.vt = (const uint16_t*)vt;
  a.bt = block_tables;
  a.maxb = maxb;
  a.items = items;
  a.n_items = n_items;
  a.r1 = r1;
  a.r2 = r2;
  a.talk = talk;
  a.out = (uint16_t*)out;
  a.H = H;
  a.G = G;
  a.BS = BS;
  a.window = window;
  a.scale = scale;
  a.part_keys = n_parts > 1 ? part_keys : 32;
  a.n_parts = n_parts > 1 ? n_parts : 1;
  a.pml = pml;
  a.po = po;
  // two heads per wave, up to eight waves: two waves per SIMD overlap one's MFMAs with the other's
  // vector work (measured against four heads per wave at 16 heads: see the design notes)
#define K8S_WIN(NDC, NV) launch_win_mfma<NDC, NV, 2>(a, s)
  if (D == 64 && V == 64) return K8S_WIN(2, 4);
  if (D == 64 && V == 128) return K8S_WIN(2, 8);
  if (D == 128 && V == 64) return K8S_WIN(4, 4);
  return K8S_WIN(4, 8);
#undef K8S_WIN
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
