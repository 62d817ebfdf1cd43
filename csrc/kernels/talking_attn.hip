// Paged attention with a logarithmic distance bias, a softmax sink and weights mixed across heads
// after the softmax ("talking heads"), for bf16 and fp32 models, over the paged cache layouts of
// the other attention kernels (K [page, Hkv, P, D], V [page, Hkv, D, P]).
//
//   s_g(i, j) = q_g(i) . k_c(g)(j) * scale - r1_g * ln(1 + r2_g * (i - j))         c(g) = g / (H / Hkv)
//   w_g(i, j) = exp(s_g(i, j)) / (exp(sink_g) + sum_j' exp(s_g(i, j')))             j in the window
//   o_h(i)    = gate_h(i) * sum_j (sum_g talk[h, g] w_g(i, j)) v_c(h)(j)
//
// The mix needs every head's NORMALISED weight of a key, so a row is done by one 256-thread
// workgroup for all heads, in two passes over the visible keys in chunks that fit LDS: pass 1
// forms the scores and each head's running maximum and sum (online across chunks); pass 2 forms
// the scores again (a row whose keys fit one chunk keeps them in LDS instead), turns them into
// final weights, mixes them over heads in LDS and accumulates the values in registers (thread =
// output element (head, value dim), up to MAXO per thread).  Scores: one thread per (kv head, key)
// reads the key row once, in 16-byte pieces, for all query heads of the group (q as fp32 in LDS,
// read as broadcasts).  Scores, weights, sums and the accumulator are fp32 for both element types.
// A row knows its block-table row and position, so prompt chunks and decode rows are one launch.
#include "common.h"

namespace {

constexpr int TA_MAXO = 32;   // output elements per thread: H * vdim <= 256 * TA_MAXO
constexpr int TA_MAXG = 16;   // query heads per kv head

template <typename T> struct Vec8 {};
template <> struct Vec8<bf16> {
  static __device__ __forceinline__ void load(const bf16* p, float (&f)[8]) {
    const bf16x8 t = ld8(p);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (float)t[j];
  }
};
template <> struct Vec8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&f)[8]) {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
    f[0] = a[0]; f[1] = a[1]; f[2] = a[2]; f[3] = a[3];
    f[4] = b[0]; f[5] = b[1]; f[6] = b[2]; f[7] = b[3];
  }
};

// scores of keys lo + c0 .. lo + c0 + n - 1 for all heads -> sc[h * CH + i]
template <typename T>
__device__ __forceinline__ void ta_scores(const float* __restrict__ qs, float* __restrict__ sc,
                                          const T* __restrict__ k_cache, const int* __restrict__ bt, int H, int Hkv,
                                          int D, int P, int CH, int pos, int key0, int n, float scale,
                                          const float* __restrict__ r1, const float* __restrict__ r2) {
  const int G = H / Hkv;
  for (int idx = threadIdx.x; idx < Hkv * n; idx += 256) {
    const int c = idx / n, i = idx - c * n;
    const int key = key0 + i;
    const T* kp = k_cache + (((int64_t)bt[key / P] * Hkv + c) * P + key % P) * D;
    float acc[TA_MAXG];
#pragma unroll
    for (int g = 0; g < TA_MAXG; ++g) acc[g] = 0.f;
    for (int d0 = 0; d0 < D; d0 += 8) {
      float kv[8];
      Vec8<T>::load(kp + d0, kv);
#pragma unroll
      for (int g = 0; g < TA_MAXG; ++g) {
        if (g < G) {
          const float* qh = qs + (c * G + g) * D + d0;
#pragma unroll
          for (int j = 0; j < 8; ++j) acc[g] += qh[j] * kv[j];
        }
      }
    }
    const float dist = (float)(pos - key);
#pragma unroll
    for (int g = 0; g < TA_MAXG; ++g) {
      if (g < G) {
        const int h = c * G + g;
        sc[h * CH + i] = acc[g] * scale - r1[h] * log1pf(r2[h] * dist);
      }
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void talking_attn_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ row_seq,
    const int* __restrict__ row_pos, const T* __restrict__ gate, int64_t gate_stride, T* __restrict__ out,
    int64_t out_stride, int H, int Hkv, int D, int vdim, int P, float scale, int window,
    const float* __restrict__ sinks, const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ talk, int CH) {
  extern __shared__ float sm[];
  float* qs = sm;                    // [H][D]
  float* sc = qs + H * D;            // [H][CH] scores, then final weights
  float* pm = sc + H * CH;           // [H][CH] mixed weights
  float* tk = pm + H * CH;           // [H][H]
  float* mh = tk + H * H;            // [H] running maximum
  float* lh = mh + H;                // [H] running sum
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int pos = row_pos[t];
  const int NO = H * vdim;
  T* orow = out + t * out_stride;
  if (pos < 0) {   // padding row: no keys
    for (int o = tid; o < NO; o += 256) orow[o] = (T)0.f;
    return;
  }
  const int* bt = block_tables + (int64_t)row_seq[t] * bt_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_vis = pos - lo + 1;
  for (int i = tid; i < H * D; i += 256) qs[i] = (float)q[t * q_stride + i];
  for (int i = tid; i < H * H; i += 256) tk[i] = talk[i];
  for (int i = tid; i < H; i += 256) {
    mh[i] = -__builtin_inff();
    lh[i] = 0.f;
  }
  __syncthreads();
  const bool one = n_vis <= CH;
  // ---- pass 1: maximum and sum per head
  for (int c0 = 0; c0 < n_vis; c0 += CH) {
    const int n = min(CH, n_vis - c0);
    ta_scores<T>(qs, sc, k_cache, bt, H, Hkv, D, P, CH, pos, lo + c0, n, scale, r1, r2);
    __syncthreads();
    for (int h = wave; h < H; h += 4) {
      float cm = -__builtin_inff();
      for (int i = lane; i < n; i += 64) cm = fmaxf(cm, sc[h * CH + i]);
      cm = wave_max(cm);
      const float m_old = mh[h], m_new = fmaxf(m_old, cm);
      float ps = 0.f;
      for (int i = lane; i < n; i += 64) ps += expf(sc[h * CH + i] - m_new);
      ps = wave_sum(ps);
      if (lane == 0) {
        lh[h] = lh[h] * expf(m_old - m_new) + ps;   // first chunk: exp(-inf) = 0
        mh[h] = m_new;
      }
    }
    __syncthreads();
  }
  if (tid < H) {   // the sink joins the denominator once
    const float sk = sinks != nullptr ? sinks[tid] : -__builtin_inff();
    const float m_new = fmaxf(mh[tid], sk);
    lh[tid] = lh[tid] * expf(mh[tid] - m_new) + (sinks != nullptr ? expf(sk - m_new) : 0.f);
    mh[tid] = m_new;
  }
  __syncthreads();
  // ---- pass 2: final weights, mixed over heads, times the values
  float acc[TA_MAXO];
#pragma unroll
  for (int u = 0; u < TA_MAXO; ++u) acc[u] = 0.f;
  const int G = H / Hkv;
  for (int c0 = 0; c0 < n_vis; c0 += CH) {
    const int n = min(CH, n_vis - c0);
    if (!one) {
      ta_scores<T>(qs, sc, k_cache, bt, H, Hkv, D, P, CH, pos, lo + c0, n, scale, r1, r2);
      __syncthreads();
    }
    for (int idx = tid; idx < H * n; idx += 256) {
      const int h = idx / n, i = idx - h * n;
      sc[h * CH + i] = expf(sc[h * CH + i] - mh[h]) / lh[h];
    }
    __syncthreads();
    for (int idx = tid; idx < H * n; idx += 256) {
      const int h = idx / n, i = idx - h * n;
      float a = 0.f;
      for (int g = 0; g < H; ++g) a += tk[h * H + g] * sc[g * CH + i];
      pm[h * CH + i] = a;
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < TA_MAXO; ++u) {
      const int o = tid + 256 * u;
      if (o < NO) {
        const int h = o / vdim, d = o - h * vdim;
        const int c = h / G;
        const float* ph = pm + h * CH;
        float a = acc[u];
        int i = 0;
        while (i < n) {   // keys of one page are contiguous in the value cache
          const int key = lo + c0 + i;
          const int off = key % P;
          const int m = min(P - off, n - i);
          const T* vp = v_cache + (((int64_t)bt[key / P] * Hkv + c) * D + d) * P + off;
          for (int j = 0; j < m; ++j) a += ph[i + j] * (float)vp[j];
          i += m;
        }
        acc[u] = a;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int u = 0; u < TA_MAXO; ++u) {
    const int o = tid + 256 * u;
    if (o < NO) {
      float a = acc[u];
      if (gate != nullptr) a *= 1.f / (1.f + expf(-(float)gate[t * gate_stride + o / vdim]));
      orow[o] = (T)a;
    }
  }
}

}  // namespace

// q [T, H, D] (row stride q_stride, heads D apart, zero beyond the key width), gate [T, H] logits
// (row stride gate_stride, nullptr: no gate), out [T, H * vdim].  r1 / r2 / sinks fp32 [H], talk
// fp32 [H, H].
OME_API int ome_talking_attn(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                             const int* block_tables, int bt_stride, const int* row_seq, const int* row_pos,
                             const void* gate, int64_t gate_stride, void* out, int64_t out_stride, int T, int H,
                             int Hkv, int D, int vdim, int P, float scale, int window, const float* sinks,
                             const float* r1, const float* r2, const float* talk, int f32, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || Hkv <= 0 || H % Hkv || H / Hkv > TA_MAXG || D <= 0 || D % 8 || vdim <= 0 || vdim > D ||
      H * vdim > 256 * TA_MAXO || P <= 0 || r1 == nullptr || r2 == nullptr || talk == nullptr)
    return -2;
  // LDS: q + talk + stats fixed, the rest split between the two weight buffers
  const int fixed = H * D + H * H + 2 * H;
  const int budget = 160 * 1024 / 4 - 64;
  if (fixed + 2 * H * 16 > budget) return -3;
  int CH = (budget - fixed) / (2 * H);   // keys per chunk: a whole window when it fits, at most 2048
  const int span = window > 0 ? window : 2048;
  if (CH > span) CH = span;
  if (CH > 2048) CH = 2048;
  const size_t lds = (size_t)(fixed + 2 * H * CH) * sizeof(float);
#define TA_LAUNCH(TT)                                                                                                \
  do {                                                                                                               \
    static bool big_ = false; /* once: allow the largest dynamic LDS block */                                       \
    if (lds > 64 * 1024 && !big_) {                                                                                \
      hipError_t e_ = hipFuncSetAttribute((const void*)talking_attn_kernel<TT>,                                                \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                \
      if (e_ != hipSuccess) return (int)e_;                                                                        \
      big_ = true;                                                                                                 \
    }                                                                                                              \
    talking_attn_kernel<TT><<<T, 256, lds, stream>>>(                                                                \
        (const TT*)q, q_stride, (const TT*)k_cache, (const TT*)v_cache, block_tables, bt_stride, row_seq, row_pos,   \
        (const TT*)gate, gate_stride, (TT*)out, out_stride, H, Hkv, D, vdim, P, scale, window, sinks, r1, r2, talk,  \
        CH);                                                                                                         \
  } while (0)
  if (f32) TA_LAUNCH(float);
  else TA_LAUNCH(bf16);
#undef TA_LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}
