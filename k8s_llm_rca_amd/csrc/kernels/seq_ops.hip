// Sequence-state kernels for models whose layers carry state from token to
// token besides the paged cache: sinusoidal positions, the short causal
// convolution in front of a sublayer, the minGRU recurrence, the
// post-sublayer norm of the fp32 residual, and the latent projections' norms
// with the paged latent write.
//
// A step's rows are grouped in SEGMENTS: consecutive rows of one sequence
// (one decode token, or a portion of a prompt).  seg_row0[n_seg + 1] are the
// row offsets, seg_pos0[s] the position of the segment's first token in its
// sequence, seg_slot[s] the sequence's state slot, row_seg[T] the segment of
// every row.  State of a slot is read only when seg_pos0 > 0: a fresh slot needs
// no clearing.
//
// The residual stream, every norm, the recurrence and its gates are fp32
// whatever the activation type; TA (activations) and TW (weights) are bf16
// (stored as uint16_t) or float.
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldf(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldf<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldf<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void stf(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void stf<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void stf<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

// x[t] = embed[ids[t]] + sinusoid(pos[t]): entry 2i = sin(p f_i), 2i+1 = cos(p f_i),
// f_i = base^(-2i / W).  The angle is formed in double so that it is exact to
// fp32 at any position.
template <typename TW>
__global__ void __launch_bounds__(256) embed_sinpos_kernel(const int* __restrict__ ids, const int* __restrict__ pos,
                                                           const TW* __restrict__ embed, float* __restrict__ x, int W,
                                                           float base) {
  const int t = blockIdx.x;
  const size_t e0 = (size_t)ids[t] * W;
  const double p = (double)pos[t], lb = log((double)base);
  for (int c = threadIdx.x; c < W; c += 256) {
    const double ang = p * exp(-(double)(2 * (c >> 1)) / (double)W * lb);
    const float pe = (float)((c & 1) ? cos(ang) : sin(ang));
    x[(size_t)t * W + c] = ldf(embed, e0 + c) + pe;
  }
}

// h[r] = x[r] + sum_j w[:, j] * in(r - taps + 1 + j): rows before the segment come
// from the slot's tail (the last taps - 1 inputs), zeros before the sequence.
// tail: [n_slots][taps - 1][W] fp32, entry k = the input at position pos0 - (taps - 1) + k.
template <typename TW, typename TA>
__global__ void __launch_bounds__(256) canon_conv_kernel(const float* __restrict__ x, const TW* __restrict__ w,
                                                         const float* __restrict__ tail,
                                                         const int* __restrict__ row_seg,
                                                         const int* __restrict__ seg_row0,
                                                         const int* __restrict__ seg_pos0,
                                                         const int* __restrict__ seg_slot, TA* __restrict__ h, int W,
                                                         int taps) {
  const int r = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int sg = row_seg[r], r0 = seg_row0[sg], p0 = seg_pos0[sg];
  const float* tl = tail + (size_t)seg_slot[sg] * (taps - 1) * W;
  const float xv = x[(size_t)r * W + c];
  float acc = xv;
  for (int j = 0; j < taps; ++j) {
    const int d = taps - 1 - j;          // this tap reads the input d rows back
    const int rr = r - d;
    float v;
    if (rr >= r0) {
      v = d == 0 ? xv : x[(size_t)rr * W + c];
    } else {
      const int back = r0 - rr;          // 1 .. taps - 1 inputs before the segment
      v = (p0 - back >= 0) ? tl[(size_t)(taps - 1 - back) * W + c] : 0.f;
    }
    acc = fmaf(ldf(w, (size_t)c * taps + j), v, acc);
  }
  stf(h, (size_t)r * W + c, acc);
}

// After the convolution of a step: the slot's tail becomes the last taps - 1
// inputs up to the segment's end (old entries shift down when the segment is
// shorter than the tail; zeros stand for positions before the sequence).
__global__ void __launch_bounds__(256) canon_tail_kernel(const float* __restrict__ x, float* __restrict__ tail,
                                                         const int* __restrict__ seg_row0,
                                                         const int* __restrict__ seg_pos0,
                                                         const int* __restrict__ seg_slot, int W, int taps) {
  constexpr int kMaxTail = 15;
  const int sg = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= W) return;
  const int r0 = seg_row0[sg], n = seg_row0[sg + 1] - r0, p0 = seg_pos0[sg], nt = taps - 1;
  float* tl = tail + (size_t)seg_slot[sg] * nt * W;
  float nv[kMaxTail];
#pragma unroll
  for (int k = 0; k < kMaxTail; ++k) {
    if (k < nt) {
      const int back = nt - k;           // new entry k = the input `back` tokens before the new end
      const int rr = r0 + n - back;
      if (rr >= r0) {
        nv[k] = x[(size_t)rr * W + c];
      } else {
        const int b0 = r0 - rr;          // inputs before the segment
        nv[k] = (p0 - b0 >= 0) ? tl[(size_t)(nt - b0) * W + c] : 0.f;
      }
    }
  }
#pragma unroll
  for (int k = 0; k < kMaxTail; ++k)
    if (k < nt) tl[(size_t)k * W + c] = nv[k];
}

// minGRU over a segment, one thread per channel: zug [T][3 C] fp32 holds the
// projections (z | u | g) without biases.  z = sigmoid(zr + bz), u = ur + bu,
// candidate = u + 1/2 (u >= 0) or sigmoid(u); S <- (1 - z) S + z cand;
// y = S * silu(g).  state [n_slots][C] fp32.
template <typename TW, typename TA>
__global__ void __launch_bounds__(256) mingru_scan_kernel(const float* __restrict__ zug, const TW* __restrict__ bz,
                                                          const TW* __restrict__ bu, float* __restrict__ state,
                                                          const int* __restrict__ seg_row0,
                                                          const int* __restrict__ seg_pos0,
                                                          const int* __restrict__ seg_slot, TA* __restrict__ y,
                                                          int C) {
  const int sg = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int r0 = seg_row0[sg], r1 = seg_row0[sg + 1];
  float* st = state + (size_t)seg_slot[sg] * C + c;
  float S = seg_pos0[sg] > 0 ? *st : 0.f;
  const float vbz = ldf(bz, c), vbu = ldf(bu, c);
#pragma unroll 4
  for (int r = r0; r < r1; ++r) {
    const float* row = zug + (size_t)r * 3 * C;
    const float z = 1.f / (1.f + expf(-(row[c] + vbz)));
    const float u = row[C + c] + vbu;
    const float g = row[2 * C + c];
    const float cand = u >= 0.f ? u + 0.5f : 1.f / (1.f + expf(-u));
    S = (1.f - z) * S + z * cand;
    stf(y, (size_t)r * C + c, S * (g / (1.f + expf(-g))));
  }
  *st = S;
}

// The same recurrence for long segments, parallel over time: the rows are cut in
// chunks ([n][4] int32: segment, first row, rows, index of the segment's first
// chunk).  Pass 1 reduces every chunk to (A, B) with S_out = A S_in + B and saves
// the segment's incoming state; pass 2 folds the earlier chunks' (A, B) into the
// chunk's S_in, runs the chunk step by step as the sequential kernel does, and
// the segment's last chunk stores the state.
__device__ __forceinline__ void mingru_gates(const float* row, int C, int c, float vbz, float vbu, float& z,
                                             float& cand) {
  z = 1.f / (1.f + expf(-(row[c] + vbz)));
  const float u = row[C + c] + vbu;
  cand = u >= 0.f ? u + 0.5f : 1.f / (1.f + expf(-u));
}

template <typename TW>
__global__ void __launch_bounds__(256) mingru_chunk_sum_kernel(const float* __restrict__ zug, const TW* __restrict__ bz,
                                                               const TW* __restrict__ bu,
                                                               const float* __restrict__ state,
                                                               const int* __restrict__ chunks,
                                                               const int* __restrict__ seg_pos0,
                                                               const int* __restrict__ seg_slot,
                                                               float* __restrict__ ab, float* __restrict__ s0, int C) {
  const int ck = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int sg = chunks[ck * 4], r0 = chunks[ck * 4 + 1], n = chunks[ck * 4 + 2], first = chunks[ck * 4 + 3];
  const float vbz = ldf(bz, c), vbu = ldf(bu, c);
  float A = 1.f, B = 0.f;
#pragma unroll 4
  for (int r = r0; r < r0 + n; ++r) {
    float z, cand;
    mingru_gates(zug + (size_t)r * 3 * C, C, c, vbz, vbu, z, cand);
    A *= 1.f - z;
    B = (1.f - z) * B + z * cand;
  }
  ab[((size_t)ck * 2) * C + c] = A;
  ab[((size_t)ck * 2 + 1) * C + c] = B;
  if (ck == first) s0[(size_t)sg * C + c] = seg_pos0[sg] > 0 ? state[(size_t)seg_slot[sg] * C + c] : 0.f;
}

template <typename TW, typename TA>
__global__ void __launch_bounds__(256) mingru_chunk_apply_kernel(const float* __restrict__ zug,
                                                                 const TW* __restrict__ bz, const TW* __restrict__ bu,
                                                                 float* __restrict__ state,
                                                                 const int* __restrict__ chunks,
                                                                 const int* __restrict__ seg_row0,
                                                                 const int* __restrict__ seg_slot,
                                                                 const float* __restrict__ ab,
                                                                 const float* __restrict__ s0, TA* __restrict__ y,
                                                                 int C) {
  const int ck = blockIdx.x, c = blockIdx.y * 256 + threadIdx.x;
  if (c >= C) return;
  const int sg = chunks[ck * 4], r0 = chunks[ck * 4 + 1], n = chunks[ck * 4 + 2], first = chunks[ck * 4 + 3];
  float S = s0[(size_t)sg * C + c];
  for (int j = first; j < ck; ++j) S = ab[((size_t)j * 2) * C + c] * S + ab[((size_t)j * 2 + 1) * C + c];
  const float vbz = ldf(bz, c), vbu = ldf(bu, c);
#pragma unroll 4
  for (int r = r0; r < r0 + n; ++r) {
    const float* row = zug + (size_t)r * 3 * C;
    float z, cand;
    mingru_gates(row, C, c, vbz, vbu, z, cand);
    const float g = row[2 * C + c];
    S = (1.f - z) * S + z * cand;
    stf(y, (size_t)r * C + c, S * (g / (1.f + expf(-g))));
  }
  if (r0 + n == seg_row0[sg + 1]) state[(size_t)seg_slot[sg] * C + c] = S;
}

// x <- unit_rms(alpha x + y) * (1 + w), in place on the fp32 residual.
// y == nullptr: the sublayer is absent (x <- unit_rms(alpha x) * (1 + w)); with `out` the normed
// row goes there instead of x (the model's last norm, alpha = 1: x is left as it is).
template <typename TY, typename TW, typename TO>
__global__ void __launch_bounds__(256) postnorm_kernel(float* __restrict__ x, const TY* __restrict__ y,
                                                       const TW* __restrict__ w, TO* __restrict__ out, int W,
                                                       float alpha, float eps) {
  __shared__ float scratch[16];
  const size_t o = (size_t)blockIdx.x * W;
  float ss = 0.f;
  for (int c = threadIdx.x; c < W; c += 256) {
    float v = x[o + c];
    if (y || alpha != 1.f) {
      v = y ? fmaf(alpha, v, ldf(y, o + c)) : alpha * v;
      x[o + c] = v;
    }
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(ss / (float)W + eps);
  for (int c = threadIdx.x; c < W; c += 256) {
    const float v = x[o + c] * inv * (1.f + ldf(w, c));
    if (out) stf(out, o + c, v); else x[o + c] = v;
  }
}

// One row of the joint down projection [T][ld] fp32 = (query latent | key-value
// latent): both are divided by their root mean square and scaled by a plain
// weight.  The query latent goes to cq [T][QR]; the key-value latent (KR > 0)
// to the paged latent cache at slots[t] (skipped when negative), and to its
// transposed twin cache_t when there is one.
template <typename TW, typename TA>
__global__ void __launch_bounds__(256) latent_norm_kernel(const float* __restrict__ dn, int ld,
                                                          const TW* __restrict__ wq, const TW* __restrict__ wkv,
                                                          const int* __restrict__ slots, TA* __restrict__ cq,
                                                          TA* __restrict__ cache, TA* __restrict__ cache_t, int BS,
                                                          int QR, int KR, float eps) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const float* row = dn + (size_t)t * ld;
  float ss = 0.f;
  for (int c = threadIdx.x; c < QR; c += 256) ss = fmaf(row[c], row[c], ss);
  ss = block_sum(ss, scratch);
  float inv = 1.f / sqrtf(ss / (float)QR + eps);
  for (int c = threadIdx.x; c < QR; c += 256) stf(cq, (size_t)t * QR + c, row[c] * inv * ldf(wq, c));
  if (KR <= 0) return;
  const int slot = slots[t];
  ss = 0.f;
  for (int c = threadIdx.x; c < KR; c += 256) ss = fmaf(row[QR + c], row[QR + c], ss);
  ss = block_sum(ss, scratch);
  inv = 1.f / sqrtf(ss / (float)KR + eps);
  if (slot < 0) return;
  const size_t page = slot / BS, off = slot - page * BS;
  for (int c = threadIdx.x; c < KR; c += 256) {
    const float v = row[QR + c] * inv * ldf(wkv, c);
    stf(cache, (size_t)slot * KR + c, v);
    if (cache_t) stf(cache_t, (page * KR + c) * BS + off, v);   // the transposed pages [pages][KR][BS]
  }
}

}  // namespace k8s

using namespace k8s;

// dt: 0 = bf16 activations and weights, 1 = fp32
#define K8S_DT2(dt, ...)                  \
  if ((dt) == 0) {                         \
    using TW = uint16_t;                   \
    using TA = uint16_t;                   \
    __VA_ARGS__;                                  \
  } else {                                 \
    using TW = float;                      \
    using TA = float;                      \
    __VA_ARGS__;                                  \
  }

K8S_API int k8s_embed_sinpos(const int* ids, const int* pos, const void* embed, float* x, int T, int W, float base,
                             int dt, hipStream_t s) {
  if (T <= 0) return 0;
  K8S_DT2(dt, hipLaunchKernelGGL((embed_sinpos_kernel<TW>), dim3(T), dim3(256), 0, s, ids, pos, (const TW*)embed, x,
                                  W, base));
  return (int)hipGetLastError();
}

K8S_API int k8s_canon_conv(const float* x, const void* w, float* tail, const int* row_seg, const int* seg_row0,
                           const int* seg_pos0, const int* seg_slot, void* h, int T, int n_seg, int W, int taps,
                           int dt, hipStream_t s) {
  if (taps < 1 || taps > 16) return (int)hipErrorInvalidValue;
  if (T <= 0) return 0;
  const int cb = (W + 255) / 256;
  K8S_DT2(dt, hipLaunchKernelGGL((canon_conv_kernel<TW, TA>), dim3(T, cb), dim3(256), 0, s, x, (const TW*)w, tail,
                                  row_seg, seg_row0, seg_pos0, seg_slot, (TA*)h, W, taps));
  if (taps > 1)
    hipLaunchKernelGGL(canon_tail_kernel, dim3(n_seg, cb), dim3(256), 0, s, x, tail, seg_row0, seg_pos0, seg_slot, W,
                       taps);
  return (int)hipGetLastError();
}

K8S_API int k8s_mingru_scan(const float* zug, const void* bz, const void* bu, float* state, const int* seg_row0,
                            const int* seg_pos0, const int* seg_slot, void* y, int n_seg, int C, int dt,
                            hipStream_t s) {
  if (n_seg <= 0) return 0;
  K8S_DT2(dt, hipLaunchKernelGGL((mingru_scan_kernel<TW, TA>), dim3(n_seg, (C + 255) / 256), dim3(256), 0, s, zug,
                                  (const TW*)bz, (const TW*)bu, state, seg_row0, seg_pos0, seg_slot, (TA*)y, C));
  return (int)hipGetLastError();
}

// ab: [n_chunks][2][C] fp32 scratch, s0: [n_seg][C] fp32 scratch.
K8S_API int k8s_mingru_chunked(const float* zug, const void* bz, const void* bu, float* state, const int* chunks,
                               int n_chunks, const int* seg_row0, const int* seg_pos0, const int* seg_slot,
                               float* ab, float* s0, void* y, int C, int dt, hipStream_t s) {
  if (n_chunks <= 0) return 0;
  const dim3 grid(n_chunks, (C + 255) / 256);
  K8S_DT2(dt, hipLaunchKernelGGL((mingru_chunk_sum_kernel<TW>), grid, dim3(256), 0, s, zug, (const TW*)bz,
                                 (const TW*)bu, state, chunks, seg_pos0, seg_slot, ab, s0, C));
  K8S_DT2(dt, hipLaunchKernelGGL((mingru_chunk_apply_kernel<TW, TA>), grid, dim3(256), 0, s, zug, (const TW*)bz,
                                 (const TW*)bu, state, chunks, seg_row0, seg_slot, ab, s0, (TA*)y, C));
  return (int)hipGetLastError();
}

// y_dt: type of y (0 bf16, 1 fp32, ignored when y is null); w_dt: the weight's;
// out (optional, type w_dt) receives the normed row instead of x.
K8S_API int k8s_postnorm(float* x, const void* y, int y_dt, const void* w, int w_dt, void* out, int T, int W,
                         float alpha, float eps, hipStream_t s) {
  if (T <= 0) return 0;
  if (w_dt == 0) {
    if (y_dt == 0)
      hipLaunchKernelGGL((postnorm_kernel<uint16_t, uint16_t, uint16_t>), dim3(T), dim3(256), 0, s, x,
                         (const uint16_t*)y, (const uint16_t*)w, (uint16_t*)out, W, alpha, eps);
    else
      hipLaunchKernelGGL((postnorm_kernel<float, uint16_t, uint16_t>), dim3(T), dim3(256), 0, s, x, (const float*)y,
                         (const uint16_t*)w, (uint16_t*)out, W, alpha, eps);
  } else {
    if (y_dt == 0) return (int)hipErrorInvalidValue;
    hipLaunchKernelGGL((postnorm_kernel<float, float, float>), dim3(T), dim3(256), 0, s, x, (const float*)y,
                       (const float*)w, (float*)out, W, alpha, eps);
  }
  return (int)hipGetLastError();
}

K8S_API int k8s_latent_norm(const float* dn, int ld, const void* wq, const void* wkv, const int* slots, void* cq,
                            void* cache, void* cache_t, int BS, int T, int QR, int KR, float eps, int dt,
                            hipStream_t s) {
  if (T <= 0) return 0;
  K8S_DT2(dt, hipLaunchKernelGGL((latent_norm_kernel<TW, TA>), dim3(T), dim3(256), 0, s, dn, ld, (const TW*)wq,
                                  (const TW*)wkv, slots, (TA*)cq, (TA*)cache, (TA*)cache_t, BS, QR, KR, eps));
  return (int)hipGetLastError();
}
