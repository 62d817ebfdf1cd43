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

// ------------------------------------------------------------------------------------------
// Prompt chunks on the matrix cores (bf16).  One workgroup = 16 consecutive query rows of one
// sequence (a quarter / half of a prefill work item) x ALL heads; wave w owns the HPW consecutive
// heads from w * HPW (heads of one kv head share its key and value fragments).  Keys go by in tiles of 32 (two pages):
//
//   pass 1   per head: S^T = K Q^T (MFMA 16x16x32; lane (n, g) holds row n, keys 16X + 4g + i),
//            bias, mask, running maximum and sum per row -> with the sink, m and 1 / l to LDS.
//   pass 2   per key tile, all waves in step:
//            (a) per head: S^T again, the FINAL weights p = exp2(s - m) / l as bf16 into
//                Pb[column = (key slot, row)][head]          (head = the next product's k index)
//            (b) the mix as a matrix product: P'[h, column] = sum_g talk[h, g] Pb[column, g]
//                (MFMA, M = 16 heads h, K = 32 heads g, N = the 16 rows of one key slot), written as
//                bf16 into Pm[head][row][key slot]
//            (c) per head: O^T += V^T P'^T with the values of the head's own kv head (the key
//                slots are in the order the value fragment cat(page A keys 4g.., page B keys 4g..)
//                has them, so Pm rows are read as 16-byte B fragments).
//
// The weights are final before they are mixed, so the accumulator is never rescaled.  Scores,
// maxima and sums are fp32 (log2 domain); weights enter the two products as bf16, like the weights
// of every MFMA attention kernel here; talk is taken as bf16 (what a 16-bit checkpoint stores).
// ------------------------------------------------------------------------------------------
namespace {

__device__ __forceinline__ f32x4 ta_mfma(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ bf16x8 ta_cat44(bf16x4 a, bf16x4 b) {
  return bf16x8{a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
}

__device__ __forceinline__ bf16x8 ta_lds8(const bf16* p) {   // 8 elements from an 8-byte aligned LDS address
  return ta_cat44(*reinterpret_cast<const bf16x4*>(p), *reinterpret_cast<const bf16x4*>(p + 4));
}

constexpr int TP_PAD = 4;   // bf16 elements of padding per LDS row: rows 72 B apart, so the 2-byte stores of 16 rows
                            // hit 16 banks; fragments are read as two 8-byte halves

template <int D, int HPW>
__global__ __launch_bounds__(512) void talking_prefill_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu_q,
    const int* __restrict__ kv_lens, const int2* __restrict__ items, const bf16* __restrict__ gate,
    int64_t gate_stride, bf16* __restrict__ out, int64_t out_stride, int H, int Hkv, int vdim, float mul, int window,
    const float* __restrict__ sinks, const float* __restrict__ r1, const float* __restrict__ r2,
    const float* __restrict__ talk, int mode, int chunk, int RT, float* __restrict__ part_ml,
    float* __restrict__ part_o) {
  // mode 0: both passes over all keys.  Split keys (single rows with long contexts: few rows, so
  // the keys of a row are spread over gridDim.z workgroups of `chunk` keys each): mode 1 = pass 1 of
  // this workgroup's keys, raw (m, l) to part_ml; mode 2 = (m, l) merged over the splits (+ sink),
  // pass 2 of this workgroup's keys, fp32 partial outputs to part_o (they simply add up: the
  // weights are final).  Partials are indexed [tile][split][head][row < RT].
  constexpr int P = 16, NB = D / 16, KS = D / 32;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int HP = (H + 31) & ~31;          // heads as a k dimension
  const int HM = (H + 15) & ~15;          // heads as an m dimension
  const int ldb = HP + TP_PAD, ldm = 32 + TP_PAD;
  bf16* Pb = reinterpret_cast<bf16*>(smem);              // [512][ldb]
  bf16* Pm = Pb + 512 * ldb;                             // [H][16][ldm]
  bf16* Tk = Pm + H * 16 * ldm;                          // [HM][ldb]
  float* ml = reinterpret_cast<float*>(Tk + HM * ldb);   // [H][16][2]: m (log2 domain), 1 / l
  const int2 it = items[blockIdx.x];
  const int s = it.x, r0 = it.y + 16 * blockIdx.y;
  const int q0 = cu_q[s];
  const int q_len = cu_q[s + 1] - q0;
  if (r0 >= q_len) return;
  const int kv_len = kv_lens[s];
  const int prefix = kv_len - q_len;
  const int G = H / Hkv;
  const int NW = blockDim.x >> 6;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = lane & 15, g = lane >> 4;
  const int r_hi = min(r0 + 16, q_len);
  const int lo0 = window > 0 ? max(0, prefix + r0 - window + 1) : 0;
  const int Z = gridDim.z, z = blockIdx.z;
  const int kv_lo = (lo0 & ~31) + (mode ? z * chunk : 0);
  const int kv_end = mode ? min(min(kv_len, prefix + r_hi), kv_lo + chunk) : min(kv_len, prefix + r_hi);
  const int64_t tile = (int64_t)blockIdx.x * gridDim.y + blockIdx.y;
  const int* bt = block_tables + (int64_t)s * bt_stride;
  const int64_t kpage = (int64_t)Hkv * P * D;
  const int r = r0 + n;                       // this lane's query row
  const bool row_ok = r < q_len;
  const int qpos = prefix + r;
  const int lo = window > 0 ? max(0, qpos - window + 1) : 0;

  const int kv0 = min(wave * HPW, H - 1) / G;
  const bool uni = wave * HPW < H && kv0 == min(wave * HPW + HPW - 1, H - 1) / G;   // one kv head for this wave
  auto load_k = [&](int kb, int kvh, bf16x8(&fa)[KS], bf16x8(&fb)[KS]) {   // lane (key n, dims 32 ks + 8 g ..)
    const int pA = bt[kb / P];
    const int pB = (kb + P < kv_len) ? bt[kb / P + 1] : pA;
    const bf16* kA = k_cache + pA * kpage + (int64_t)kvh * P * D;
    const bf16* kB = k_cache + pB * kpage + (int64_t)kvh * P * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      fa[ks] = ld8(kA + n * D + 32 * ks + 8 * g);
      fb[ks] = ld8(kB + n * D + 32 * ks + 8 * g);
    }
  };
  if (mode != 1) {
    for (int i = threadIdx.x; i < HM * ldb; i += blockDim.x) {   // talk as bf16, zero padded
      const int h = i / ldb, c = i - h * ldb;
      Tk[i] = (bf16)((h < H && c < H) ? talk[h * H + c] : 0.f);
    }
    for (int i = threadIdx.x; i < 512 * ldb; i += blockDim.x) Pb[i] = (bf16)0.f;   // (pad heads stay zero)
  }
  if (mode == 2) {   // (m, l) of every head and row over all splits
    for (int i = threadIdx.x; i < H * RT; i += blockDim.x) {
      const int head = i / RT, nn = i - head * RT;
      float m = sinks != nullptr ? sinks[head] * 1.4426950408889634f : -__builtin_inff();
      for (int zz = 0; zz < Z; ++zz) m = fmaxf(m, part_ml[(((tile * Z + zz) * H + head) * RT + nn) * 2]);
      float l = sinks != nullptr ? __builtin_amdgcn_exp2f(sinks[head] * 1.4426950408889634f - m) : 0.f;
      for (int zz = 0; zz < Z; ++zz) {
        const float* pz = part_ml + (((tile * Z + zz) * H + head) * RT + nn) * 2;
        if (pz[1] > 0.f) l += pz[1] * __builtin_amdgcn_exp2f(pz[0] - m);
      }
      ml[(head * 16 + nn) * 2] = (m == -__builtin_inff()) ? 0.f : m;
      ml[(head * 16 + nn) * 2 + 1] = l > 0.f ? 1.f / l : 0.f;
    }
  }

  // ---- pass 1: key tiles outside, this wave's heads inside, so that heads of one kv head share the
  // key fragments (a wave owns HPW consecutive heads)
  if (mode != 2) {
    bf16x8 qf[HPW][KS];
    float m_i[HPW], l_i[HPW], b1[HPW], b2[HPW];
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      const int head = min(wave * HPW + j, H - 1);
      const bf16* qr = q + (int64_t)(q0 + min(r, q_len - 1)) * q_stride + (int64_t)head * D;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) qf[j][ks] = ld8(qr + 32 * ks + 8 * g);
      m_i[j] = -__builtin_inff();
      l_i[j] = 0.f;
      b1[j] = r1[head];
      b2[j] = r2[head];
    }
    // the key fragments of the next tile are loaded while this one is worked on (when all heads of
    // the wave share one kv head; otherwise they are loaded in place, per kv head)
    bf16x8 na[KS], nb8[KS];
    if (uni && kv_lo < kv_end) load_k(kv_lo, kv0, na, nb8);
    for (int kb = kv_lo; kb < kv_end; kb += 32) {
      bf16x8 ka[KS], kb8[KS];
      int kv_prev = -1;
      if (uni) {
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
          ka[ks] = na[ks];
          kb8[ks] = nb8[ks];
        }
        if (kb + 32 < kv_end) load_k(kb + 32, kv0, na, nb8);
        kv_prev = kv0;
      }
#pragma unroll
      for (int j = 0; j < HPW; ++j) {
        const int head = wave * HPW + j;
        if (head < H) {
          const int kvh = head / G;
          if (kvh != kv_prev) {
            load_k(kb, kvh, ka, kb8);
            kv_prev = kvh;
          }
          f32x4 sc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            sc[0] = ta_mfma(ka[ks], qf[j][ks], sc[0]);
            sc[1] = ta_mfma(kb8[ks], qf[j][ks], sc[1]);
          }
          float mt = -__builtin_inff();
#pragma unroll
          for (int X = 0; X < 2; ++X)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = kb + 16 * X + 4 * g + i;
              const bool ok = row_ok && key <= qpos && key >= lo;
              const float v =
                  ok ? sc[X][i] * mul - b1[j] * __log2f(1.f + b2[j] * (float)(qpos - key)) : -__builtin_inff();
              sc[X][i] = v;
              mt = fmaxf(mt, v);
            }
          mt = group4_max(mt);
          const float m_new = fmaxf(m_i[j], mt);
          const float m_use = (m_new == -__builtin_inff()) ? 0.f : m_new;
          float rs = 0.f;
#pragma unroll
          for (int X = 0; X < 2; ++X)
#pragma unroll
            for (int i = 0; i < 4; ++i) rs += __builtin_amdgcn_exp2f(sc[X][i] - m_use);
          rs = group4_sum(rs);
          l_i[j] = l_i[j] * __builtin_amdgcn_exp2f(m_i[j] - m_use) + rs;
          m_i[j] = m_new;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      const int head = wave * HPW + j;
      if (head < H) {
        if (mode == 1) {
          if (g == 0 && n < RT) {
            float* pz = part_ml + (((tile * Z + z) * H + head) * RT + n) * 2;
            pz[0] = m_i[j];
            pz[1] = l_i[j];
          }
        } else {
          float mm = m_i[j], ll = l_i[j];
          if (sinks != nullptr) {
            const float sk = sinks[head] * 1.4426950408889634f;
            const float m_new = fmaxf(mm, sk);
            ll = ll * __builtin_amdgcn_exp2f(mm - m_new) + __builtin_amdgcn_exp2f(sk - m_new);
            mm = m_new;
          }
          if (g == 0) {
            ml[(head * 16 + n) * 2] = (mm == -__builtin_inff()) ? 0.f : mm;
            ml[(head * 16 + n) * 2 + 1] = ll > 0.f ? 1.f / ll : 0.f;
          }
        }
      }
    }
  }
  if (mode == 1) return;
  __syncthreads();

  // ---- pass 2
  f32x4 o[HPW][NB];
#pragma unroll
  for (int j = 0; j < HPW; ++j)
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) o[j][nb] = f32x4{0.f, 0.f, 0.f, 0.f};
  // When all heads of the wave share one kv head (uni), its loads run ahead of their use: the key
  // fragments of the NEXT tile are asked for right after (a) has used this tile's (same registers,
  // in flight during (b) and (c)), the value fragments of this tile right after the first barrier (in
  // flight during the mix).  Otherwise fragments are loaded where they are used, per kv head.
  constexpr bool VPRE = HPW * D <= 256;   // (4 heads x 128 dims of accumulators leave no registers for the values)
  bf16x8 ka[KS], kb8[KS];
  if (uni && kv_lo < kv_end) load_k(kv_lo, kv0, ka, kb8);
  for (int kb = kv_lo; kb < kv_end; kb += 32) {
    const int pA = bt[kb / P];
    const int pB = (kb + P < kv_len) ? bt[kb / P + 1] : pA;
    // (a) final weights of this wave's heads
    {
      int kv_prev = uni ? kv0 : -1;
#pragma unroll
      for (int j = 0; j < HPW; ++j) {
        const int head = wave * HPW + j;
        if (head < H) {
          const int kvh = head / G;
          if (kvh != kv_prev) {
            load_k(kb, kvh, ka, kb8);
            kv_prev = kvh;
          }
          const bf16* qr = q + (int64_t)(q0 + min(r, q_len - 1)) * q_stride + (int64_t)head * D;
          f32x4 sc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
#pragma unroll
          for (int ks = 0; ks < KS; ++ks) {
            const bf16x8 qv = ld8(qr + 32 * ks + 8 * g);
            sc[0] = ta_mfma(ka[ks], qv, sc[0]);
            sc[1] = ta_mfma(kb8[ks], qv, sc[1]);
          }
          const float b1 = r1[head], b2 = r2[head];
          const float m = ml[(head * 16 + n) * 2], il = ml[(head * 16 + n) * 2 + 1];
#pragma unroll
          for (int X = 0; X < 2; ++X)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              const int key = kb + 16 * X + 4 * g + i;
              const bool ok = row_ok && key <= qpos && key >= lo;
              const float v = sc[X][i] * mul - b1 * __log2f(1.f + b2 * (float)(qpos - key));
              const float p = ok ? __builtin_amdgcn_exp2f(v - m) * il : 0.f;
              Pb[((8 * g + 4 * X + i) * 16 + n) * ldb + head] = (bf16)p;
            }
        }
      }
    }
    if (uni && kb + 32 < kv_end) load_k(kb + 32, kv0, ka, kb8);   // the next tile's keys
    __syncthreads();
    bf16x8 vpre[VPRE ? NB : 1];
    if (VPRE && uni) {
      const bf16* vA = v_cache + pA * kpage + (int64_t)kv0 * D * P;
      const bf16* vB = v_cache + pB * kpage + (int64_t)kv0 * D * P;
#pragma unroll
      for (int nb = 0; nb < NB; ++nb)
        vpre[nb] = ta_cat44(ld4(vA + (16 * nb + n) * P + 4 * g), ld4(vB + (16 * nb + n) * P + 4 * g));
    }
    // (b) mix over heads: one key slot (16 rows) per product column block
    for (int t = wave; t < 32; t += NW) {
      for (int mt = 0; mt < HM / 16; ++mt) {
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
        for (int ks = 0; ks < HP / 32; ++ks)
          acc = ta_mfma(ta_lds8(Tk + (16 * mt + n) * ldb + 32 * ks + 8 * g),
                        ta_lds8(Pb + (16 * t + n) * ldb + 32 * ks + 8 * g), acc);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int h = 16 * mt + 4 * g + i;
          if (h < H) Pm[(h * 16 + n) * ldm + t] = (bf16)acc[i];
        }
      }
    }
    __syncthreads();
    // (c) values: a value fragment is loaded once per kv head and feeds all its heads of this wave
    {
      bf16x8 pb[HPW];
#pragma unroll
      for (int j = 0; j < HPW; ++j) {
        const int head = min(wave * HPW + j, H - 1);
        pb[j] = ta_lds8(Pm + (head * 16 + n) * ldm + 8 * g);
      }
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        const int dim = 16 * nb + n;
        bf16x8 va;
        int kv_prev = -1;
        if constexpr (VPRE) {
          if (uni) {
            va = vpre[nb];
            kv_prev = kv0;
          }
        }
#pragma unroll
        for (int j = 0; j < HPW; ++j) {
          const int head = wave * HPW + j;
          if (head < H) {
            const int kvh = head / G;
            if (kvh != kv_prev) {
              const bf16* vA = v_cache + pA * kpage + (int64_t)kvh * D * P;
              const bf16* vB = v_cache + pB * kpage + (int64_t)kvh * D * P;
              va = ta_cat44(ld4(vA + dim * P + 4 * g), ld4(vB + dim * P + 4 * g));
              kv_prev = kvh;
            }
            o[j][nb] = ta_mfma(va, pb[j], o[j][nb]);
          }
        }
      }
    }
    // (the next tile's (a) writes Pb only, and its (b) follows a barrier after this tile's (c))
  }
  // ---- epilogue: O^T lane (row n, dims 16 nb + 4 g + i), times the head's gate
  if (mode == 2) {
    if (row_ok && n < RT) {
#pragma unroll
      for (int j = 0; j < HPW; ++j) {
        const int head = wave * HPW + j;
        if (head < H) {
          float* po = part_o + (((tile * Z + z) * H + head) * RT + n) * D;
#pragma unroll
          for (int nb = 0; nb < NB; ++nb)
            *reinterpret_cast<f32x4*>(po + 16 * nb + 4 * g) = o[j][nb];
        }
      }
    }
    return;
  }
  if (row_ok) {
#pragma unroll
    for (int j = 0; j < HPW; ++j) {
      const int head = wave * HPW + j;
      if (head < H) {
        const float gt = gate != nullptr
                             ? 1.f / (1.f + __expf(-(float)gate[(int64_t)(q0 + r) * gate_stride + head])) : 1.f;
        bf16* orow = out + (int64_t)(q0 + r) * out_stride + (int64_t)head * vdim;
#pragma unroll
        for (int nb = 0; nb < NB; ++nb)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int dim = 16 * nb + 4 * g + i;
            if (dim < vdim) orow[dim] = (bf16)(o[j][nb][i] * gt);
          }
      }
    }
  }
}

// out[b, h * vdim + d] = gate(b, h) * sum over splits of part_o[b][z][h][d]   (single rows: RT = 1)
__global__ __launch_bounds__(256) void talking_combine_kernel(const float* __restrict__ part_o, int Z, int H, int D,
                                                              int vdim, const bf16* __restrict__ gate,
                                                              int64_t gate_stride, bf16* __restrict__ out,
                                                              int64_t out_stride) {
  const int64_t b = blockIdx.x;
  const int o = blockIdx.y * 256 + threadIdx.x;   // one output element per thread
  if (o < H * vdim) {
    const int h = o / vdim, d = o - h * vdim;
    float a = 0.f;
    for (int z = 0; z < Z; ++z) a += part_o[(((b * Z + z) * H + h)) * D + d];
    if (gate != nullptr) a *= 1.f / (1.f + __expf(-(float)gate[b * gate_stride + h]));
    out[b * out_stride + o] = (bf16)a;
  }
}

}  // namespace

// items int32 [n_items, 2] = (sequence, first row) of `item_rows`-row work items (a multiple of 16);
// sequence s owns query rows cu_q[s] .. cu_q[s + 1] at positions kv_lens[s] - q_len ...; bf16 only.
OME_API int ome_talking_prefill(const void* q, int64_t q_stride, const void* k_cache, const void* v_cache,
                                const int* block_tables, int bt_stride, const int* cu_q, const int* kv_lens,
                                const int* items, int n_items, int item_rows, const void* gate, int64_t gate_stride,
                                void* out, int64_t out_stride, int H, int Hkv, int D, int vdim, int P, float scale,
                                int window, const float* sinks, const float* r1, const float* r2, const float* talk,
                                int splits, int chunk, float* part_ml, float* part_o, hipStream_t stream) {
  // splits > 1 (item_rows must be 16, every sequence brings ONE row: decode): keys in `splits`
  // pieces of `chunk` (a multiple of 32) per row; part_ml fp32 [n_items, splits, H, 2], part_o fp32
  // [n_items, splits, H, D]
  if (n_items <= 0) return 0;
  if (splits > 1 && (item_rows != 16 || chunk <= 0 || chunk % 32 || part_ml == nullptr || part_o == nullptr)) return -2;
  if (P != 16 || H <= 0 || Hkv <= 0 || H % Hkv || vdim <= 0 || vdim > D || item_rows <= 0 || item_rows % 16 ||
      (q_stride & 7) || r1 == nullptr || r2 == nullptr || talk == nullptr)
    return -2;
  const int hpw = D == 256 ? 2 : 4;
  const int NW = (H + hpw - 1) / hpw;
  if (NW > 8) return -3;   // (8 waves: the accumulators of HPW heads fit the registers of 2 waves per SIMD)
  const int HP = (H + 31) & ~31, HM = (H + 15) & ~15, ldb = HP + TP_PAD, ldm = 32 + TP_PAD;
  const size_t lds = (size_t)(512 * ldb + H * 16 * ldm + HM * ldb) * 2 + (size_t)H * 16 * 2 * 4;
  if (lds > 160 * 1024) return -3;
  const dim3 grid(n_items, item_rows / 16), gridz(n_items, 1, splits > 1 ? splits : 1);
  const float mul = scale * 1.4426950408889634f;
#define TP_LAUNCH(DD, HH)                                                                                            \
  do {                                                                                                               \
    static bool big_ = false;                                                                                        \
    if (lds > 64 * 1024 && !big_) {                                                                                  \
      hipError_t e_ = hipFuncSetAttribute((const void*)talking_prefill_kernel<DD, HH>,                               \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);                   \
      if (e_ != hipSuccess) return (int)e_;                                                                          \
      big_ = true;                                                                                                   \
    }                                                                                                                \
    if (splits > 1) {                                                                                                \
      for (int md = 1; md <= 2; ++md)                                                                                \
        talking_prefill_kernel<DD, HH><<<gridz, 64 * NW, md == 1 ? 0 : lds, stream>>>(                               \
            (const bf16*)q, q_stride, (const bf16*)k_cache, (const bf16*)v_cache, block_tables, bt_stride, cu_q,     \
            kv_lens, (const int2*)items, (const bf16*)gate, gate_stride, (bf16*)out, out_stride, H, Hkv, vdim, mul,  \
            window, sinks, r1, r2, talk, md, chunk, 1, part_ml, part_o);                                             \
      talking_combine_kernel<<<dim3(n_items, (H * vdim + 255) / 256), 256, 0, stream>>>(part_o, splits, H, DD, vdim, (const bf16*)gate,            \
                                                          gate_stride, (bf16*)out, out_stride);                      \
    } else {                                                                                                         \
      talking_prefill_kernel<DD, HH><<<grid, 64 * NW, lds, stream>>>(                                                \
          (const bf16*)q, q_stride, (const bf16*)k_cache, (const bf16*)v_cache, block_tables, bt_stride, cu_q,       \
          kv_lens, (const int2*)items, (const bf16*)gate, gate_stride, (bf16*)out, out_stride, H, Hkv, vdim, mul,    \
          window, sinks, r1, r2, talk, 0, 0, 16, nullptr, nullptr);                                                  \
    }                                                                                                                \
  } while (0)
  if (D == 64) TP_LAUNCH(64, 4);
  else if (D == 128) TP_LAUNCH(128, 4);
  else if (D == 256) TP_LAUNCH(256, 2);
  else return -2;
#undef TP_LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}
