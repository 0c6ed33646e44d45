// Attention over a paged LATENT cache (one vector of R numbers per token, shared
// by every head): the keys' and values' up-projections are moved to the query and
// output side, so a head's query is qa[h] = W_uk[h]^T q[h] (R numbers), its
// score against token j is scale * qa[h] . c_j, and its output in latent space
// is sum_j p_j c_j; the caller applies W_uv[h] afterwards.  All heads of a token
// read the same keys once.  Causal softmax in fp32; the per-head output gate
// sigmoid(gate[t][h]) is applied here (it commutes with W_uv).
//
// Rows are addressed through the step's segments (seq_ops.hip): row r of segment
// s is the token at position seg_pos0[s] + r - seg_row0[s] and sees keys 0 .. that
// position, read through block table row s ([n_seg][maxb] pages of BS tokens).
#include "common.h"

namespace k8s {

template <typename T>
__device__ __forceinline__ float ldc(const T* p, size_t i);
template <>
__device__ __forceinline__ float ldc<float>(const float* p, size_t i) { return p[i]; }
template <>
__device__ __forceinline__ float ldc<uint16_t>(const uint16_t* p, size_t i) { return bf2f(p[i]); }
template <typename T>
__device__ __forceinline__ void sto(T* p, size_t i, float v);
template <>
__device__ __forceinline__ void sto<float>(float* p, size_t i, float v) { p[i] = v; }
template <>
__device__ __forceinline__ void sto<uint16_t>(uint16_t* p, size_t i, float v) { p[i] = f2bf(v); }

constexpr int kKT = 32;       // keys per tile
constexpr int kMaxAcc = 8;    // outputs per thread and head group

// Any H and R, fp32 arithmetic on the vector pipes: the reference form (fp32
// models, and shapes the MFMA kernels do not take).  One workgroup per row;
// heads in groups of HG with HG * R <= 256 * kMaxAcc.
// LDS: q[HG][R] | ct[kKT][R + 1] | sc[HG][kKT] | m[HG] l[HG] al[HG]
template <typename TC, typename TO>
__global__ void __launch_bounds__(256) latent_attn_rows_kernel(
    const float* __restrict__ qa, const TC* __restrict__ cache, const int* __restrict__ bt, int maxb,
    const int* __restrict__ row_seg, const int* __restrict__ seg_row0, const int* __restrict__ seg_pos0,
    const float* __restrict__ gate, int ldg, TO* __restrict__ out, int row_base, int H, int R, int BS, int HG,
    float scale) {
  extern __shared__ float smem[];
  float* q = smem;
  float* ct = q + HG * R;
  float* sc = ct + kKT * (R + 1);
  float* m = sc + HG * kKT;
  float* l = m + HG;
  float* al = l + HG;
  const int r = row_base + blockIdx.x, tid = threadIdx.x, lane = tid & 63, wv = tid >> 6;
  const int sg = row_seg[r];
  const int ctx = seg_pos0[sg] + (r - seg_row0[sg]) + 1;
  const int* pages = bt + (size_t)sg * maxb;
  for (int h0 = 0; h0 < H; h0 += HG) {
    const int hg = min(HG, H - h0), no = hg * R;
    for (int i = tid; i < no; i += 256) q[i] = qa[((size_t)r * H + h0) * R + i];
    if (tid < hg) {
      m[tid] = -INFINITY;
      l[tid] = 0.f;
    }
    float acc[kMaxAcc];
#pragma unroll
    for (int i = 0; i < kMaxAcc; ++i) acc[i] = 0.f;
    for (int k0 = 0; k0 < ctx; k0 += kKT) {
      const int nk = min(kKT, ctx - k0);
      __syncthreads();
      for (int i = tid; i < kKT * R; i += 256) {
        const int j = i / R, c = i - j * R, kp = k0 + j;
        float v = 0.f;
        if (j < nk) v = ldc(cache, ((size_t)pages[kp / BS] * BS + kp % BS) * R + c);
        ct[j * (R + 1) + c] = v;
      }
      __syncthreads();
      for (int i = tid; i < hg * kKT; i += 256) {
        const int h = i / kKT, j = i - h * kKT;
        float s = -INFINITY;
        if (j < nk) {
          s = 0.f;
          const float* qh = q + h * R;
          const float* cj = ct + j * (R + 1);
          for (int c = 0; c < R; ++c) s = fmaf(qh[c], cj[c], s);
          s *= scale;
        }
        sc[i] = s;
      }
      __syncthreads();
      for (int h = wv; h < hg; h += 4) {      // one wave per head: kKT <= 64 scores
        const float s = lane < kKT ? sc[h * kKT + lane] : -INFINITY;
        const float mo = m[h], mn = fmaxf(mo, wave_max(s));
        const float p = lane < nk ? expf(s - mn) : 0.f;
        const float ps = wave_sum(p);
        if (lane < kKT) sc[h * kKT + lane] = p;
        if (lane == 0) {
          const float a = expf(mo - mn);      // 0 on the first tile (mo = -inf)
          al[h] = a;
          l[h] = l[h] * a + ps;
          m[h] = mn;
        }
      }
      __syncthreads();
#pragma unroll
      for (int i = 0; i < kMaxAcc; ++i) {
        const int o = tid + i * 256;
        if (o < no) {
          const int h = o / R, c = o - h * R;
          float a = acc[i] * al[h];
          const float* ph = sc + h * kKT;
          for (int j = 0; j < nk; ++j) a = fmaf(ph[j], ct[j * (R + 1) + c], a);
          acc[i] = a;
        }
      }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < kMaxAcc; ++i) {
      const int o = tid + i * 256;
      if (o < no) {
        const int h = o / R;
        const float g = 1.f / (1.f + expf(-gate[(size_t)r * ldg + h0 + h]));
        sto(out, ((size_t)r * H + h0) * R + o, acc[i] / l[h] * g);
      }
    }
    __syncthreads();
  }
}

}  // namespace k8s

using namespace k8s;

// Rows row_base .. row_base + n_rows of the step.  dt: 0 = bf16 cache and output, 1 = fp32.
K8S_API int k8s_latent_attn_rows(const float* qa, const void* cache, const int* bt, int maxb, const int* row_seg,
                                 const int* seg_row0, const int* seg_pos0, const float* gate, int ldg, void* out,
                                 int row_base, int n_rows, int H, int R, int BS, float scale, int dt,
                                 hipStream_t s) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || R <= 0 || R > 256 * kMaxAcc) return (int)hipErrorInvalidValue;
  int HG = (256 * kMaxAcc) / R;
  if (HG > 64) HG = 64;
  if (HG > H) HG = H;
  const size_t lds = sizeof(float) * ((size_t)HG * R + (size_t)kKT * (R + 1) + (size_t)HG * kKT + 3 * HG);
  if (lds > 160 * 1024) return (int)hipErrorInvalidValue;
  if (dt == 0) {
    auto k = latent_attn_rows_kernel<uint16_t, uint16_t>;
    if (lds > 48 * 1024) hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(k, dim3(n_rows), dim3(256), lds, s, qa, (const uint16_t*)cache, bt, maxb, row_seg, seg_row0,
                       seg_pos0, gate, ldg, (uint16_t*)out, row_base, H, R, BS, HG, scale);
  } else {
    auto k = latent_attn_rows_kernel<float, float>;
    if (lds > 48 * 1024) hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(k, dim3(n_rows), dim3(256), lds, s, qa, (const float*)cache, bt, maxb, row_seg, seg_row0,
                       seg_pos0, gate, ldg, (float*)out, row_base, H, R, BS, HG, scale);
  }
  return (int)hipGetLastError();
}
