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

namespace k8s {

// ---------------------------------------------------------------------------
// MFMA form (bf16): v_mfma_f32_16x16x32_bf16, one wave per work item, no LDS.
//
// The latents are cached twice: c [pages][BS][R] (a key's R numbers contiguous:
// the QK^T operand) and ct [pages][R][BS] (8 consecutive keys of one latent
// column contiguous: the PV operand), as the K / transposed-V pages of the
// head-wise attention kernels.  A wave owns MT tiles of 16 query rows; a tile is
// TPM consecutive tokens x HC heads (HC = min(H, 16), TPM = 16 / HC), so all its
// rows read the same keys.  Keys go in chunks of 32 (never across a page:
// BS % 32 == 0).  Swapped QK^T (S^T = C Q^T): a lane owns ONE query row
// (lane & 15) and 8 of its key scores; MFMA row rho of key tile t holds key
// 8 (rho >> 2) + 4 t + (rho & 3), so lane quarter h ends with keys 8h .. 8h + 7,
// the k-slots of the PV operand: P moves from accumulator to operand in place.
//
// Items ([n][4] int32: segment, first row, tokens, position of the first row's
// token) are made on the host from the step's segments.  SPLIT (decode rows):
// grid.y partitions of `part` keys write unnormalised partials which
// latent_reduce merges -- the partition borders depend on the key index only,
// never on the batch.  Otherwise (prompt portions) a wave walks every key its
// rows see and writes the gated, normalised output.
constexpr float kLog2e = 1.4426950408889634f;

struct LatArgs {
  const uint16_t* qa;     // [T][H][R] bf16
  const uint16_t* c;      // [pages][BS][R]
  const uint16_t* ct;     // [pages][R][BS]
  const int* bt;
  int maxb;
  const int* items;
  int n_items;
  const float* gate;
  int ldg;
  uint16_t* out;          // [T][H][R]
  float* part_o;          // [T][H][n_parts][R]
  float* part_ml;         // [T][H][n_parts][2]
  int n_parts, part;
  int H, HC, TPM, BS;
  float scale_log2;
};

__device__ __forceinline__ bf16x8 ld16(const uint16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }

template <int NR, int MT, bool SPLIT>
__global__ void __launch_bounds__(256) latent_attn_mfma_kernel(LatArgs a) {
  constexpr int R = NR * 32, ND = R / 16;
  const int lane = threadIdx.x & 63, r = lane & 15, h = lane >> 4;
  // workgroups go round-robin over the 8 XCDs, each with its own L2: give every XCD a contiguous
  // range of items (neighbouring token groups of the same sequences read the same latent pages)
  const int per = gridDim.x >> 3;
  const int blk = (gridDim.x & 7) == 0 ? (blockIdx.x & 7) * per + (blockIdx.x >> 3) : blockIdx.x;
  const int item = blk * 4 + (threadIdx.x >> 6);
  if (item >= a.n_items) return;
  const int sg = a.items[item * 4], row0 = a.items[item * 4 + 1], ntok = a.items[item * 4 + 2],
            pos0 = a.items[item * 4 + 3];
  const int hc = blockIdx.z;
  int k_begin = 0, k_end = pos0 + ntok;
  if constexpr (SPLIT) {
    k_begin = blockIdx.y * a.part;
    k_end = min(k_end, k_begin + a.part);
    if (k_begin >= k_end) return;
  }
  // this lane's query row in every tile
  const int tl = r / a.HC, hl = r - tl * a.HC, head = hc * a.HC + hl;
  bf16x8 qf[MT][NR];
  int limit[MT];
  f32x4 o[MT][ND];
  float m[MT], l[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int ti = mt * a.TPM + tl;
    const bool valid = tl < a.TPM && ti < ntok && head < a.H;
    limit[mt] = valid ? min(pos0 + ti + 1, k_end) : 0;
    const uint16_t* qp = a.qa + ((size_t)(row0 + (valid ? ti : 0)) * a.H + (valid ? head : 0)) * R;
#pragma unroll
    for (int cc = 0; cc < NR; ++cc) {
      qf[mt][cc] = ld16(qp + 32 * cc + 8 * h);
      if (!valid)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[mt][cc][j] = (__bf16)0.f;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) o[mt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[mt] = -INFINITY;
    l[mt] = 0.f;
  }
  const int* pages = a.bt + (size_t)sg * a.maxb;
  for (int kb = k_begin & ~31; kb < k_end; kb += 32) {
    const int page = pages[kb / a.BS], off = kb % a.BS;
    const uint16_t* cp = a.c + (size_t)page * a.BS * R;
    const uint16_t* tp = a.ct + (size_t)page * R * a.BS;
    bf16x8 kf[2][NR];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = off + 8 * (r >> 2) + 4 * t + (r & 3);
#pragma unroll
      for (int cc = 0; cc < NR; ++cc) kf[t][cc] = ld16(cp + (size_t)key * R + 32 * cc + 8 * h);
    }
    bf16x8 pf[MT];
    float ar[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float p[8];
      float cmax = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int cc = 0; cc < NR; ++cc) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][cc], qf[mt][cc], s, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb + 8 * h + 4 * t + i;
          const float v = (key < limit[mt] && key >= k_begin) ? s[i] * a.scale_log2 : -INFINITY;
          p[4 * t + i] = v;
          cmax = fmaxf(cmax, v);
        }
      }
      cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
      cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
      const float mnew = fmaxf(m[mt], cmax);
      const float alpha = (mnew == -INFINITY) ? 1.f : exp2f(m[mt] - mnew);
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = (mnew == -INFINITY) ? 0.f : exp2f(p[j] - mnew);
        psum += e;
        pf[mt][j] = (__bf16)e;
      }
      l[mt] = l[mt] * alpha + psum;
      m[mt] = mnew;
#pragma unroll
      for (int i = 0; i < 4; ++i) ar[mt][i] = __shfl(alpha, 4 * h + i, 64);
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
      const bf16x8 vf = ld16(tp + (size_t)(16 * dt + r) * a.BS + off + 8 * h);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[mt][dt][i] *= ar[mt][i];
        o[mt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[mt], vf, o[mt][dt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float lt = l[mt];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = 4 * h + i;                       // the query row of accumulator element i
      const int qtl = q / a.HC, qhl = q - qtl * a.HC, qhead = hc * a.HC + qhl, ti = mt * a.TPM + qtl;
      const float lq = __shfl(lt, q, 64), mq = __shfl(m[mt], q, 64);
      if (!(qtl < a.TPM && ti < ntok && qhead < a.H)) continue;
      const size_t rh = (size_t)(row0 + ti) * a.H + qhead;
      if constexpr (SPLIT) {
        const size_t pi = rh * a.n_parts + blockIdx.y;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) a.part_o[pi * R + 16 * dt + r] = o[mt][dt][i];
        if (r == 0) {
          a.part_ml[pi * 2] = mq;
          a.part_ml[pi * 2 + 1] = lq;
        }
      } else {
        const float g = 1.f / (1.f + expf(-a.gate[(size_t)(row0 + ti) * a.ldg + qhead]));
        const float sc = lq > 0.f ? g / lq : 0.f;
#pragma unroll
        for (int dt = 0; dt < ND; ++dt) a.out[rh * R + 16 * dt + r] = f2bf(o[mt][dt][i] * sc);
      }
    }
  }
}

// Prompt portions: the four waves of a workgroup own four consecutive items of ONE
// segment (the host pads every segment's items to a multiple of four with empty
// ones), so they read the same keys.  A chunk's operand fragments do not depend on
// the item: kf[t][cc] and vf[dt] are loaded from global memory once per workgroup
// (a quarter by each wave), parked in LDS in fragment order -- slot f holds the 64
// lanes' 16 bytes, so writes and reads are conflict-free -- and read back by all
// four waves.  Two buffers: chunk i + 1 is fetched into registers while chunk i
// is computed, and written after it; one barrier per chunk.
template <int NR, int MT, int OCC>
__global__ void __launch_bounds__(256, OCC) latent_attn_mfma_lds_kernel(LatArgs a) {
  constexpr int R = NR * 32, ND = R / 16, NF = 2 * NR + ND, NFW = NF / 4;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  bf16x8* frag = reinterpret_cast<bf16x8*>(lds_raw);          // [2][NF][64]
  __shared__ int kend_s[4];
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6, r = lane & 15, h = lane >> 4;
  // ... and the LAST items of the range first: they see the most keys, so the short ones fill the tail
  const int per = gridDim.x >> 3;
  const int blk = (gridDim.x & 7) == 0 ? (blockIdx.x & 7) * per + (per - 1 - (blockIdx.x >> 3))
                                       : gridDim.x - 1 - blockIdx.x;
  const int item0 = blk * 4;
  if (item0 >= a.n_items) return;                              // whole workgroup
  const int item = item0 + wv;
  const int sg = a.items[item0 * 4];
  const int row0 = a.items[item * 4 + 1], ntok = a.items[item * 4 + 2], pos0 = a.items[item * 4 + 3];
  const int hc = blockIdx.z;
  if (lane == 0) kend_s[wv] = ntok > 0 ? pos0 + ntok : 0;
  __syncthreads();
  const int k_end = max(max(kend_s[0], kend_s[1]), max(kend_s[2], kend_s[3]));
  const int tl = r / a.HC, hl = r - tl * a.HC, head = hc * a.HC + hl;
  bf16x8 qf[MT][NR];
  int limit[MT];
  f32x4 o[MT][ND];
  float m[MT], l[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int ti = mt * a.TPM + tl;
    const bool valid = tl < a.TPM && ti < ntok && head < a.H;
    limit[mt] = valid ? pos0 + ti + 1 : 0;
    const uint16_t* qp = a.qa + ((size_t)(row0 + (valid ? ti : 0)) * a.H + (valid ? head : 0)) * R;
#pragma unroll
    for (int cc = 0; cc < NR; ++cc) {
      qf[mt][cc] = ld16(qp + 32 * cc + 8 * h);
      if (!valid)
#pragma unroll
        for (int j = 0; j < 8; ++j) qf[mt][cc][j] = (__bf16)0.f;
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) o[mt][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
    m[mt] = -INFINITY;
    l[mt] = 0.f;
  }
  const int* pages = a.bt + (size_t)sg * a.maxb;
  // this wave's share of a chunk's fragments: f = wv + 4 i
  bf16x8 pre[NFW];
  auto fetch = [&](int kb) {
    const int page = pages[kb / a.BS], off = kb % a.BS;
    const uint16_t* cp = a.c + (size_t)page * a.BS * R;
    const uint16_t* tp = a.ct + (size_t)page * R * a.BS;
#pragma unroll
    for (int i = 0; i < NFW; ++i) {
      const int f = wv + 4 * i;
      if (f < 2 * NR) {
        const int t = f / NR, cc = f - t * NR;
        const int key = off + 8 * (r >> 2) + 4 * t + (r & 3);
        pre[i] = ld16(cp + (size_t)key * R + 32 * cc + 8 * h);
      } else {
        const int dt = f - 2 * NR;
        pre[i] = ld16(tp + (size_t)(16 * dt + r) * a.BS + off + 8 * h);
      }
    }
  };
  auto park = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NFW; ++i) frag[((size_t)buf * NF + wv + 4 * i) * 64 + lane] = pre[i];
  };
  if (k_end > 0) {
    fetch(0);
    park(0);
  }
  int buf = 0;
  for (int kb = 0; kb < k_end; kb += 32, buf ^= 1) {
    __syncthreads();
    const bool more = kb + 32 < k_end;
    if (more) fetch(kb + 32);
    const bf16x8* fb = frag + (size_t)buf * NF * 64 + lane;
    f32x4 s[MT][2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) s[mt][t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int cc = 0; cc < NR; ++cc) {
        const bf16x8 kf = fb[(t * NR + cc) * 64];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          s[mt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[mt][cc], s[mt][t], 0, 0, 0);
      }
    }
    bf16x8 pf[MT];
    float ar[MT][4];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float p[8];
      float cmax = -INFINITY;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kb + 8 * h + 4 * t + i;
          const float v = key < limit[mt] ? s[mt][t][i] * a.scale_log2 : -INFINITY;
          p[4 * t + i] = v;
          cmax = fmaxf(cmax, v);
        }
      cmax = fmaxf(cmax, __shfl_xor(cmax, 16, 64));
      cmax = fmaxf(cmax, __shfl_xor(cmax, 32, 64));
      const float mnew = fmaxf(m[mt], cmax);
      const float alpha = (mnew == -INFINITY) ? 1.f : exp2f(m[mt] - mnew);
      float psum = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float e = (mnew == -INFINITY) ? 0.f : exp2f(p[j] - mnew);
        psum += e;
        pf[mt][j] = (__bf16)e;
      }
      l[mt] = l[mt] * alpha + psum;
      m[mt] = mnew;
#pragma unroll
      for (int i = 0; i < 4; ++i) ar[mt][i] = __shfl(alpha, 4 * h + i, 64);
    }
#pragma unroll
    for (int dt = 0; dt < ND; ++dt) {
      const bf16x8 vf = fb[(2 * NR + dt) * 64];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) o[mt][dt][i] *= ar[mt][i];
        o[mt][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pf[mt], vf, o[mt][dt], 0, 0, 0);
      }
    }
    if (more) park(buf ^ 1);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    float lt = l[mt];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = 4 * h + i;
      const int qtl = q / a.HC, qhl = q - qtl * a.HC, qhead = hc * a.HC + qhl, ti = mt * a.TPM + qtl;
      const float lq = __shfl(lt, q, 64);
      if (!(qtl < a.TPM && ti < ntok && qhead < a.H)) continue;
      const size_t rh = (size_t)(row0 + ti) * a.H + qhead;
      const float g = 1.f / (1.f + expf(-a.gate[(size_t)(row0 + ti) * a.ldg + qhead]));
      const float sc = lq > 0.f ? g / lq : 0.f;
#pragma unroll
      for (int dt = 0; dt < ND; ++dt) a.out[rh * R + 16 * dt + r] = f2bf(o[mt][dt][i] * sc);
    }
  }
}

// Merge of the key partitions of decode rows: one workgroup per (row, head).
// A row at position p has ceil((p + 1) / part) partitions.
__global__ void __launch_bounds__(128) latent_reduce_kernel(const float* __restrict__ part_o,
                                                            const float* __restrict__ part_ml,
                                                            const int* __restrict__ positions,
                                                            const float* __restrict__ gate, int ldg,
                                                            uint16_t* __restrict__ out, int H, int R, int n_parts,
                                                            int part) {
  const int row = blockIdx.x / H, head = blockIdx.x - row * H;
  const size_t rh = (size_t)row * H + head;
  const int np = min(n_parts, positions[row] / part + 1);
  float mx = -INFINITY;
  for (int p = 0; p < np; ++p) mx = fmaxf(mx, part_ml[(rh * n_parts + p) * 2]);
  float lsum = 0.f;
  for (int p = 0; p < np; ++p) lsum += exp2f(part_ml[(rh * n_parts + p) * 2] - mx) * part_ml[(rh * n_parts + p) * 2 + 1];
  const float g = 1.f / (1.f + expf(-gate[(size_t)row * ldg + head]));
  for (int c = threadIdx.x; c < R; c += 128) {
    float acc = 0.f;
    for (int p = 0; p < np; ++p)
      acc = fmaf(exp2f(part_ml[(rh * n_parts + p) * 2] - mx), part_o[(rh * n_parts + p) * R + c], acc);
    out[rh * R + c] = f2bf(acc / lsum * g);
  }
}

template <int NR>
static int launch_lat(const LatArgs& a, int split, int mt2, int n_head_chunks, hipStream_t s) {
  int nblk = (a.n_items + 3) / 4;
  if (nblk > 8) nblk = (nblk + 7) & ~7;   // a multiple of the XCD count (the kernels' item remap)
  const dim3 grid(nblk, split ? a.n_parts : 1, n_head_chunks);
  if (split) {
    hipLaunchKernelGGL((latent_attn_mfma_kernel<NR, 1, true>), grid, dim3(256), 0, s, a);
    return (int)hipGetLastError();
  }
  if (a.n_items % 4) return (int)hipErrorInvalidValue;   // prompt items come in fours per segment
  constexpr size_t lds = 2 * (size_t)(4 * NR) * 64 * 16;  // two buffers of 2 NR + R / 16 fragments of 1 KiB
  // tiles per wave and waves per SIMD by register need: two tiles while two waves still fit a SIMD
  // (R <= 128), one tile and two waves at R = 192 / 256, one and one above
  constexpr int MT = NR <= 4 ? 2 : 1, OCC = NR <= 8 ? 2 : 1;
  auto k = latent_attn_mfma_lds_kernel<NR, MT, OCC>;
  if (lds > 48 * 1024 && hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds))
    return (int)hipGetLastError();
  hipLaunchKernelGGL(k, grid, dim3(256), lds, s, a);
  return (int)hipGetLastError();
}

}  // namespace k8s

// 0: the MFMA kernels do not take latent rank R; else the tiles per wave for prompt portions (2 up to R = 128).
K8S_API int k8s_latent_attn_mfma_ok(int R) {
  switch (R) {
    case 32: case 64: case 96: case 128: return 2;
    case 192: case 256: case 384: case 512: return 1;
    default: return 0;
  }
}

// split = 1: decode rows (items of one token), partials + merge into out; `positions` [T] are the
// rows' positions and n_rows the number of decode rows (the first rows of the step).
// split = 0: prompt portions, items of up to tiles * (16 / min(H, 16)) tokens.
K8S_API int k8s_latent_attn_mfma(const void* qa, const void* c, const void* ct, const int* bt, int maxb,
                                 const int* items, int n_items, const float* gate, int ldg, void* out,
                                 float* part_o, float* part_ml, int n_parts, int part, const int* positions,
                                 int n_rows, int H, int R, int BS, float scale, int split, int tiles,
                                 hipStream_t s) {
  if (n_items <= 0) return 0;
  if (!k8s_latent_attn_mfma_ok(R) || BS % 32 || H <= 0 || (split && part % 32)) return (int)hipErrorInvalidValue;
  k8s::LatArgs a;
  a.qa = (const uint16_t*)qa; a.c = (const uint16_t*)c; a.ct = (const uint16_t*)ct; a.bt = bt; a.maxb = maxb;
  a.items = items; a.n_items = n_items; a.gate = gate; a.ldg = ldg; a.out = (uint16_t*)out;
  a.part_o = part_o; a.part_ml = part_ml; a.n_parts = n_parts; a.part = part;
  a.H = H; a.HC = H < 16 ? H : 16; a.TPM = 16 / a.HC; a.BS = BS; a.scale_log2 = scale * k8s::kLog2e;
  const int nhc = (H + a.HC - 1) / a.HC, mt2 = (!split && tiles == 2);
  int rc;
  switch (R / 32) {
    case 1: rc = k8s::launch_lat<1>(a, split, mt2, nhc, s); break;
    case 2: rc = k8s::launch_lat<2>(a, split, mt2, nhc, s); break;
    case 3: rc = k8s::launch_lat<3>(a, split, mt2, nhc, s); break;
    case 4: rc = k8s::launch_lat<4>(a, split, mt2, nhc, s); break;
    case 6: rc = k8s::launch_lat<6>(a, split, mt2, nhc, s); break;
    case 8: rc = k8s::launch_lat<8>(a, split, mt2, nhc, s); break;
    case 12: rc = k8s::launch_lat<12>(a, split, mt2, nhc, s); break;
    case 16: rc = k8s::launch_lat<16>(a, split, mt2, nhc, s); break;
    default: return (int)hipErrorInvalidValue;
  }
  if (rc || !split) return rc;
  hipLaunchKernelGGL(k8s::latent_reduce_kernel, dim3(n_rows * H), dim3(128), 0, s, part_o, part_ml, positions, gate, ldg,
                     (uint16_t*)out, H, R, n_parts, part);
  return (int)hipGetLastError();
}
