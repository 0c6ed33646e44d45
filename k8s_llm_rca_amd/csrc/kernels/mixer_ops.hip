// Recurrent mixers over segments: a short causal convolution with bias and
// activation (its last taps - 1 inputs are per-sequence state), the selective
// scan of a diagonal state-space layer, and retention (linear attention with a
// fixed decay per head, rotary positions, per-head unit norm and output gate).
//
// Segments as in seq_ops.hip: seg_row0[n_seg + 1] row offsets, seg_pos0[s] the
// position of the segment's first token, seg_slot[s] the sequence's state slot,
// row_seg[T] the segment of every row.  State of a slot is read only when
// seg_pos0 > 0.  All recurrences, their decays, step sizes and gates are fp32;
// TA is the activation type (bf16 as uint16_t, or float).
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldm(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldm<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldm<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void stm(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void stm<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void stm<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

__device__ __forceinline__ float silu_f(float v) { return v / (1.f + expf(-v)); }

// out[r][c] = act(b[c] + sum_j w[c][j] * in(r - (taps - 1 - j))): the last column is the current
// token's tap.  Inputs before the segment come from the slot's tail (entry k = the input at
// position pos0 - (taps - 1) + k), zeros before the sequence.  x rows have stride xs.
template <typename TA>
__global__ void __launch_bounds__(256) short_conv_kernel(const TA* __restrict__ x, int xs, const float* __restrict__ w,
                                                         const float* __restrict__ b, const float* __restrict__ tail,
                                                         const int* __restrict__ row_seg,
                                                         const int* __restrict__ seg_row0,
                                                         const int* __restrict__ seg_pos0,
                                                         const int* __restrict__ seg_slot, TA* __restrict__ out, int C,
                                                         int taps, int act) {
  const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int sg = row_seg[r], r0 = seg_row0[sg], p0 = seg_pos0[sg];
  const float* tl = tail + (size_t)seg_slot[sg] * (taps - 1) * C;
  float acc = b ? b[c] : 0.f;
  for (int j = 0; j < taps; ++j) {
    const int rr = r - (taps - 1 - j);
    float v;
    if (rr >= r0) {
      v = ldm(x, (size_t)rr * xs + c);
    } else {
      const int back = r0 - rr;          // 1 .. taps - 1 inputs before the segment
      v = (p0 - back >= 0) ? tl[(size_t)(taps - 1 - back) * C + c] : 0.f;
    }
    acc = fmaf(w[(size_t)c * taps + j], v, acc);
  }
  stm(out, (size_t)r * C + c, act ? silu_f(acc) : acc);
}

// After the convolution of a step: the slot's tail becomes the last taps - 1 inputs up to the
// segment's end (old entries shift down when the segment is shorter than the tail).
template <typename TA>
__global__ void __launch_bounds__(256) short_conv_tail_kernel(const TA* __restrict__ x, int xs, float* __restrict__ tail,
                                                              const int* __restrict__ seg_row0,
                                                              const int* __restrict__ seg_pos0,
                                                              const int* __restrict__ seg_slot, int C, int taps) {
  constexpr int kMaxTail = 15;
  const int sg = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = seg_row0[sg], n = seg_row0[sg + 1] - r0, p0 = seg_pos0[sg], nt = taps - 1;
  float* tl = tail + (size_t)seg_slot[sg] * nt * C;
  float nv[kMaxTail];
#pragma unroll
  for (int k = 0; k < kMaxTail; ++k) {
    if (k < nt) {
      const int back = nt - k;           // new entry k = the input `back` tokens before the new end
      const int rr = r0 + n - back;
      if (rr >= r0) {
        nv[k] = ldm(x, (size_t)rr * xs + c);
      } else {
        const int b0 = r0 - rr;          // inputs before the segment
        nv[k] = (p0 - b0 >= 0) ? tl[(size_t)(nt - b0) * C + c] : 0.f;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kMaxTail; ++k)
    if (k < nt) tl[(size_t)k * C + c] = nv[k];
}

// Selective scan, one thread per channel, the channel's N states in registers:
//   dt = softplus(dtp[r][c] + dt_bias[c]);  S[n] <- exp(dt A[c][n]) S[n] + dt x B[r][n];
//   y = (sum_n S[n] C[r][n] + D[c] x) * silu(z[r][c]).
// dbc rows (stride ds) hold B at column R and C at column R + N, fp32.  state [slots][C][N].
template <int NMAX, typename TA>
__global__ void __launch_bounds__(128) selective_scan_kernel(const TA* __restrict__ xc, const float* __restrict__ dtp,
                                                             const float* __restrict__ dt_bias,
                                                             const float* __restrict__ dbc, int ds, int R,
                                                             const float* __restrict__ A, const float* __restrict__ Dp,
                                                             const TA* __restrict__ z, int zs, float* __restrict__ state,
                                                             const int* __restrict__ seg_row0,
                                                             const int* __restrict__ seg_pos0,
                                                             const int* __restrict__ seg_slot, TA* __restrict__ y,
                                                             int C, int N) {
  const int sg = blockIdx.x, c = blockIdx.y * 128 + threadIdx.x;
  if (c >= C) return;
  const int r0 = seg_row0[sg], r1 = seg_row0[sg + 1];
  const bool fresh = seg_pos0[sg] == 0;
  float* st = state + ((size_t)seg_slot[sg] * C + c) * N;
  float S[NMAX], Ac[NMAX];
#pragma unroll
  for (int n = 0; n < NMAX; ++n) {
    Ac[n] = n < N ? A[(size_t)c * N + n] : 0.f;
    S[n] = (n < N && !fresh) ? st[n] : 0.f;
  }
  const float Dc = Dp[c], bias = dt_bias[c];
  for (int r = r0; r < r1; ++r) {
    const float dv = dtp[(size_t)r * C + c] + bias;
    const float dt = dv > 20.f ? dv : log1pf(expf(dv));
    const float xv = ldm(xc, (size_t)r * C + c);
    const float dx = dt * xv;
    const float* Bp = dbc + (size_t)r * ds + R;
    const float* Cp = Bp + N;
    float acc = 0.f;
#pragma unroll
    for (int n = 0; n < NMAX; ++n)
      if (n < N) {
        S[n] = fmaf(expf(dt * Ac[n]), S[n], dx * Bp[n]);
        acc = fmaf(S[n], Cp[n], acc);
      }
    const float zv = ldm(z, (size_t)r * zs + c);
    stm(y, (size_t)r * C + c, (acc + Dc * xv) * silu_f(zv));
  }
#pragma unroll
  for (int n = 0; n < NMAX; ++n)
    if (n < N) st[n] = S[n];
}

// Retention, one workgroup per (segment, head), token by token.  Rows of qkvg (fp32, stride qs):
// q [H][D] | k [H][D] | v [H][V] | g [H][V].  q and k are rotated on their first `rot` entries
// (entry i with i + rot / 2; angle = pos * base^(-2 i / rot), formed in double), k is scaled by
// D^(-1/2);  S <- decay S + k v^T;  o = S^T q;  out = o / rms(o) * silu(g).
// Thread (dg, v) of NDG x V owns S[d][v] for d = dg, dg + NDG, ...  state [slots][H][D][V].
constexpr int kRetDpt = 64;
template <typename TA>
__global__ void __launch_bounds__(256) retention_kernel(const float* __restrict__ qkvg, int qs,
                                                        const int* __restrict__ positions,
                                                        const float* __restrict__ decay, float* __restrict__ state,
                                                        const int* __restrict__ seg_row0,
                                                        const int* __restrict__ seg_pos0,
                                                        const int* __restrict__ seg_slot, TA* __restrict__ out, int H,
                                                        int D, int V, int rot, float base, float eps) {
  extern __shared__ float sm[];
  __shared__ float red[16];
  const int sg = blockIdx.x, hh = blockIdx.y, tid = threadIdx.x;
  const int NDG = 256 / V, half = rot >> 1;
  float* sq = sm;                 // [D]
  float* sk = sq + D;             // [D]
  float* sv = sk + D;             // [V]
  float* part = sv + V;           // [NDG][V]
  float* cs = part + NDG * V;     // [half] cos | [half] sin
  const int v = tid % V, dg = tid / V;
  const bool own = dg < NDG;
  const int r0 = seg_row0[sg], r1 = seg_row0[sg + 1];
  const bool fresh = seg_pos0[sg] == 0;
  float* st = state + ((size_t)seg_slot[sg] * H + hh) * D * V;
  const float dec = decay[hh], ks = 1.f / sqrtf((float)D);
  float S[kRetDpt];
#pragma unroll
  for (int i = 0; i < kRetDpt; ++i) {
    const int d = dg + i * NDG;
    S[i] = (own && d < D && !fresh) ? st[(size_t)d * V + v] : 0.f;
  }
  const double lb = log((double)base);
  for (int r = r0; r < r1; ++r) {
    const float* row = qkvg + (size_t)r * qs;
    __syncthreads();
    if (tid < half) {
      const double ang = (double)positions[r] * exp(-(double)(2 * tid) / (double)rot * lb);
      cs[tid] = (float)cos(ang);
      cs[half + tid] = (float)sin(ang);
    }
    __syncthreads();
    for (int d = tid; d < D; d += 256) {
      const float* q = row + hh * D;
      const float* k = row + (H + hh) * D;
      float qv, kv;
      if (d < half) {
        qv = q[d] * cs[d] - q[d + half] * cs[half + d];
        kv = k[d] * cs[d] - k[d + half] * cs[half + d];
      } else if (d < rot) {
        const int i = d - half;
        qv = q[d] * cs[i] + q[i] * cs[half + i];
        kv = k[d] * cs[i] + k[i] * cs[half + i];
      } else {
        qv = q[d];
        kv = k[d];
      }
      sq[d] = qv;
      sk[d] = kv * ks;
    }
    for (int i = tid; i < V; i += 256) sv[i] = row[2 * H * D + hh * V + i];
    __syncthreads();
    if (own) {
      const float vv = sv[v];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < kRetDpt; ++i) {
        const int d = dg + i * NDG;
        if (d < D) {
          S[i] = fmaf(dec, S[i], sk[d] * vv);
          acc = fmaf(S[i], sq[d], acc);
        }
      }
      part[dg * V + v] = acc;
    }
    __syncthreads();
    float o = 0.f;
    if (tid < V)
      for (int g = 0; g < NDG; ++g) o += part[g * V + tid];
    const float ss = block_sum(tid < V ? o * o : 0.f, red);
    if (tid < V) {
      const float gv = row[2 * H * D + H * V + hh * V + tid];
      stm(out, (size_t)r * H * V + hh * V + tid, o / sqrtf(ss / (float)V + eps) * silu_f(gv));
    }
  }
#pragma unroll
  for (int i = 0; i < kRetDpt; ++i) {
    const int d = dg + i * NDG;
    if (own && d < D) st[(size_t)d * V + v] = S[i];
  }
}

}  // namespace k8s

using namespace k8s;

#define K8S_MDT(dt, ...)   \
  if ((dt) == 0) {          \
    using TA = uint16_t;    \
    __VA_ARGS__;            \
  } else {                  \
    using TA = float;       \
    __VA_ARGS__;            \
  }

K8S_API int k8s_short_conv(const void* x, int xs, int xdt, const float* w, const float* b, float* tail,
                           const int* row_seg, const int* seg_row0, const int* seg_pos0, const int* seg_slot,
                           void* out, int T, int n_seg, int C, int taps, int act, int odt, hipStream_t s) {
  if (T <= 0) return 0;
  if (taps < 1 || taps > 16 || xdt != odt) return (int)hipErrorInvalidValue;
  const dim3 g1(T, (C + 255) / 256), g2(n_seg, (C + 255) / 256);
  K8S_MDT(odt, {
    hipLaunchKernelGGL((short_conv_kernel<TA>), g1, dim3(256), 0, s, (const TA*)x, xs, w, b, tail, row_seg, seg_row0,
                       seg_pos0, seg_slot, (TA*)out, C, taps, act);
    if (taps > 1)
      hipLaunchKernelGGL((short_conv_tail_kernel<TA>), g2, dim3(256), 0, s, (const TA*)x, xs, tail, seg_row0,
                         seg_pos0, seg_slot, C, taps);
  });
  return (int)hipGetLastError();
}

K8S_API int k8s_selective_scan(const void* xc, int dt, const float* dtp, const float* dt_bias, const float* dbc,
                               int ds, int R, const float* A, const float* D, const void* z, int zs, float* state,
                               const int* seg_row0, const int* seg_pos0, const int* seg_slot, void* y, int n_seg,
                               int C, int N, int T, hipStream_t s) {
  if (T <= 0 || n_seg <= 0) return 0;
  if (N < 1 || N > 128) return (int)hipErrorInvalidValue;
  const dim3 g(n_seg, (C + 127) / 128);
#define K8S_SCAN(NM)                                                                                              \
  K8S_MDT(dt, hipLaunchKernelGGL((selective_scan_kernel<NM, TA>), g, dim3(128), 0, s, (const TA*)xc, dtp, dt_bias, \
                                 dbc, ds, R, A, D, (const TA*)z, zs, state, seg_row0, seg_pos0, seg_slot, (TA*)y, \
                                 C, N))
  if (N <= 16) {
    K8S_SCAN(16);
  } else if (N <= 32) {
    K8S_SCAN(32);
  } else if (N <= 64) {
    K8S_SCAN(64);
  } else {
    K8S_SCAN(128);
  }
#undef K8S_SCAN
  return (int)hipGetLastError();
}

K8S_API int k8s_retention(const float* qkvg, int qs, const int* positions, const float* decay, float* state,
                          const int* seg_row0, const int* seg_pos0, const int* seg_slot, void* out, int n_seg, int H,
                          int D, int V, int rot, float base, float eps, int odt, hipStream_t s) {
  if (n_seg <= 0) return 0;
  if (V < 1 || V > 256 || rot < 0 || rot > D || (rot & 1) || rot / 2 > 256) return (int)hipErrorInvalidValue;
  const int NDG = 256 / V;
  if ((D + NDG - 1) / NDG > kRetDpt) return (int)hipErrorInvalidValue;
  const size_t lds = (size_t)(2 * D + V + NDG * V + rot) * sizeof(float);
  K8S_MDT(odt, hipLaunchKernelGGL((retention_kernel<TA>), dim3(n_seg, H), dim3(256), lds, s, qkvg, qs, positions,
                                  decay, state, seg_row0, seg_pos0, seg_slot, (TA*)out, H, D, V, rot, base, eps));
  return (int)hipGetLastError();
}
