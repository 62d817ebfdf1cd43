// Fused "QKV split -> RoPE -> paged KV-cache write" (kernels K2 + K3 of SURVEY.md §2.9).
//
// Input is the fused QKV projection output [T, (Hq + 2*Hkv) * D].  Q is rotated into a
// dense [T, Hq, D] buffer for the attention kernels; K is rotated and scattered into the
// paged K cache; V is scattered *transposed* into the paged V cache.
//
// Paged cache layouts (chosen for the MFMA attention kernels, see attention_*.hip):
//   K cache: [num_pages, Hkv, P, D]   — a page's keys are D-contiguous rows, so a lane can load
//                                       the A operand of S^T = K Q^T straight from HBM (16 B).
//   V cache: [num_pages, Hkv, D, P]   — transposed, so the A operand of O^T = V^T P^T is
//                                       P-contiguous (keys) and loads straight from HBM too.
// The cache element type is a template parameter (KVFmt in common.h): bf16, or OCP fp8
// e4m3 / e5m2 (`--kv-cache-dtype fp8*`, K15) stored as fp8(x / scale) with saturation.
// RoPE is the NeoX / HF "rotate_half" form; the cos/sin table [max_pos, rot_dim] (cos in the
// first half, sin in the second) is precomputed on the host with the model's rope scaling
// (llama3 / yarn / linear), so the kernel stays a pure streaming op (Appendix B, trig tables).
#include "common.h"

template <int D, int P, int F>
__global__ __launch_bounds__(256) void rope_qkv_cache_kernel(
    const bf16* __restrict__ qkv, int64_t qkv_stride, const int* __restrict__ positions,
    const float* __restrict__ cos_sin, int rot_dim, bf16* __restrict__ q_out,
    typename KVStore<F>::T* __restrict__ k_cache, typename KVStore<F>::T* __restrict__ v_cache,
    const int* __restrict__ slots, int Hq, int Hkv, int apply_rope, const bf16* __restrict__ q_norm_w,
    const bf16* __restrict__ k_norm_w, float qk_eps, float k_inv_scale, float v_inv_scale, int v_rowmajor) {
  const int t = blockIdx.x;
  const bf16* row = qkv + (int64_t)t * qkv_stride;
  const int pos = positions[t];
  const int slot = slots[t];
  const float* cs = cos_sin + (int64_t)pos * rot_dim;
  const int half = rot_dim >> 1;
  constexpr int DV = D / 8;  // 8-wide vectors per head row

  // ---- Q and K: optional per-head RMSNorm (Qwen3 qk-norm), then rotate ----
  // A head row is LPH = D/8 lanes (8 dims each); a wave processes 64/LPH head rows at once
  // (4 for D=128), so the 40 Q+K rows of a Llama-3 token take 3 wave-iterations, not 10, and
  // every lane of the wave is busy.  All reductions / partner shuffles stay inside a row group.
  constexpr int LPH = D / 8, HPW = 64 / LPH;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int sub = lane / LPH, l = lane % LPH, gbase = sub * LPH;
  const int nheads = Hq + Hkv;
  // grid.y splits a token's heads over several blocks (more waves in flight per CU at decode
  // batch sizes, where one 4-wave block per token leaves the kernel latency-bound)
  for (int h0 = (blockIdx.y * 4 + wave) * HPW; h0 < nheads; h0 += gridDim.y * 4 * HPW) {
    const int h = h0 + sub;
    const bool valid = h < nheads;
    const bool is_q = h < Hq;
    bf16x8 x = {};
    if (valid) x = ld8(row + (int64_t)h * D + l * 8);
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (float)x[j];
    const bf16* nw = is_q ? q_norm_w : k_norm_w;
    if (nw != nullptr) {  // wave-uniform: q_norm_w and k_norm_w are both set or both null
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += f[j] * f[j];
#pragma unroll
      for (int m = 1; m < LPH; m <<= 1) ss += __shfl_xor(ss, m);
      const float rs = rsqrtf(ss / (float)D + qk_eps);
      if (valid) {
        bf16x8 wv = ld8(nw + l * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = (float)(bf16)(f[j] * rs * (float)wv[j]);
      }
    }
    if (apply_rope) {
      const int d0 = l * 8;
      const int hl = half >> 3;  // lanes between a dim and its rotate_half partner
      const int partner = gbase + ((d0 < half) ? l + hl : l - hl);
      float g[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) g[j] = __shfl(f[j], (partner >= gbase && partner < gbase + LPH) ? partner : lane);
      if (d0 < rot_dim) {
        const int i0 = (d0 < half) ? d0 : d0 - half;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float c = cs[i0 + j], sn = cs[half + i0 + j];
          f[j] = (d0 < half) ? (f[j] * c - g[j] * sn) : (f[j] * c + g[j] * sn);
        }
      }
    }
    if (valid) {
      if (is_q) {
        bf16x8 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = (bf16)f[j];
        st8(q_out + ((int64_t)t * Hq + h) * D + l * 8, o);
      } else if (slot >= 0) {
        const int kh = h - Hq;
        const int64_t page = slot / P, off = slot % P;
        if constexpr (F != KV_BF16) {
          // quantise the bf16-rounded key (the value a bf16 cache would have held)
#pragma unroll
          for (int j = 0; j < 8; ++j) f[j] = (float)(bf16)f[j] * k_inv_scale;
        }
        kv_st8<F>(k_cache + ((page * Hkv + kh) * P + off) * D + l * 8, f);
      }
    }
  }
  // ---- V: transposed scatter into [page][kh][d][off] ----
  // lanes take CONSECUTIVE dims: one wave store then covers 64 dim rows 2*P bytes apart (2 KB,
  // 16 cache lines) instead of 64 rows 8 dims apart (64 lines), so the partial writes of a
  // token's column coalesce per line
  if (slot >= 0) {
    const int64_t page = slot / P, off = slot % P;
    const bf16* vsrc = row + (int64_t)(Hq + Hkv) * D;
    typename KVStore<F>::T* vbase = v_cache + page * Hkv * D * P + off;
    if (!v_rowmajor) {
      for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < Hkv * D; i += gridDim.y * blockDim.x) {
        const float x = (float)vsrc[i];   // i = kh * D + d
        kv_st1<F>(vbase + (int64_t)i * P, F == KV_BF16 ? x : x * v_inv_scale);
      }
    } else {   // previous mapping (8 dims per lane), kept for A/B (OME_ROPE_VMAP=1)
      for (int i = blockIdx.y * blockDim.x + threadIdx.x; i < Hkv * DV; i += gridDim.y * blockDim.x) {
        const int kh = i / DV, dv = i % DV;
        bf16x8 x = ld8(vsrc + kh * D + dv * 8);
        typename KVStore<F>::T* dst = v_cache + ((page * Hkv + kh) * D + dv * 8) * P + off;
#pragma unroll
        for (int j = 0; j < 8; ++j) kv_st1<F>(dst + j * P, F == KV_BF16 ? (float)x[j] : (float)x[j] * v_inv_scale);
      }
    }
  }
}

// Plain paged-cache write of already-projected K [T, Hkv, D] and V [T, Hkv, D] (used by the
// PD-disaggregation receiver and by tests).
template <int D, int P, int F>
__global__ void kv_cache_write_kernel(const bf16* __restrict__ k, const bf16* __restrict__ v, int64_t kv_stride,
                                      typename KVStore<F>::T* __restrict__ k_cache,
                                      typename KVStore<F>::T* __restrict__ v_cache, const int* __restrict__ slots,
                                      int Hkv, float k_inv_scale, float v_inv_scale) {
  const int t = blockIdx.x;
  const int slot = slots[t];
  if (slot < 0) return;
  const int64_t page = slot / P, off = slot % P;
  constexpr int DV = D / 8;
  constexpr bool q8 = F != KV_BF16;
  for (int i = threadIdx.x; i < Hkv * DV; i += blockDim.x) {
    const int kh = i / DV, dv = i % DV;
    bf16x8 kx = ld8(k + t * kv_stride + kh * D + dv * 8);
    float f[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = q8 ? (float)kx[j] * k_inv_scale : (float)kx[j];
    kv_st8<F>(k_cache + ((page * Hkv + kh) * P + off) * D + dv * 8, f);
    bf16x8 vx = ld8(v + t * kv_stride + kh * D + dv * 8);
    typename KVStore<F>::T* dst = v_cache + ((page * Hkv + kh) * D + dv * 8) * P + off;
#pragma unroll
    for (int j = 0; j < 8; ++j) kv_st1<F>(dst + j * P, q8 ? (float)vx[j] * v_inv_scale : (float)vx[j]);
  }
}

static int g_rope_split = 0;  // blocks per token (0 = one per 16 Q/K heads)
OME_API int ome_rope_set_split(int ny) {
  if (ny < 0 || ny > 8) return -1;
  g_rope_split = ny;
  return 0;
}

// kv_fmt: KVFmt of the cache tensors; k_scale / v_scale: dequantisation scales (fp8 only)
static const int g_rope_vmap = [] {
  const char* e = getenv("OME_ROPE_VMAP");
  return e ? atoi(e) : 0;
}();

OME_API int ome_rope_qkv_cache(const void* qkv, int64_t qkv_stride, const int* positions, const float* cos_sin,
                               int rot_dim, void* q_out, void* k_cache, void* v_cache, const int* slots, int T,
                               int Hq, int Hkv, int D, int P, int apply_rope, const void* q_norm_w,
                               const void* k_norm_w, float qk_eps, int kv_fmt, float k_scale, float v_scale,
                               hipStream_t stream) {
  if (T <= 0) return 0;
  if (D != 128 && D != 64 && D != 256) return -2;
  if (rot_dim > D || rot_dim % 16 != 0) return -3;
  if (P != 16) return -4;
  if (kv_fmt < 0 || kv_fmt > 2) return -5;
  const float ki = 1.f / k_scale, vi = 1.f / v_scale;
  // blocks per token: enough 4-wave blocks that each covers at most one 4-head group per wave
  const int per_block = 4 * (512 / D);
  // (decode batches only: 5.4 vs 6.3 us at T = 256; no gain once T fills the chip)
  int ny = g_rope_split > 0 ? g_rope_split : (T < 512 ? (Hq + Hkv + per_block - 1) / per_block : 1);
  ny = ny < 1 ? 1 : (ny > 8 ? 8 : ny);
  const dim3 grid(T, ny);
#define LAUNCH(DD, FF)                                                                                          \
  rope_qkv_cache_kernel<DD, 16, FF><<<grid, 256, 0, stream>>>(                                                    \
      (const bf16*)qkv, qkv_stride, positions, cos_sin, rot_dim, (bf16*)q_out, (KVStore<FF>::T*)k_cache,       \
      (KVStore<FF>::T*)v_cache, slots, Hq, Hkv, apply_rope, (const bf16*)q_norm_w, (const bf16*)k_norm_w,      \
      qk_eps, ki, vi, g_rope_vmap)
  if (D == 128) {
    if (kv_fmt == KV_BF16) LAUNCH(128, KV_BF16);
    else if (kv_fmt == KV_E4M3) LAUNCH(128, KV_E4M3);
    else LAUNCH(128, KV_E5M2);
  } else if (D == 256) {
    if (kv_fmt == KV_BF16) LAUNCH(256, KV_BF16);
    else if (kv_fmt == KV_E4M3) LAUNCH(256, KV_E4M3);
    else LAUNCH(256, KV_E5M2);
  } else {
    if (kv_fmt == KV_BF16) LAUNCH(64, KV_BF16);
    else if (kv_fmt == KV_E4M3) LAUNCH(64, KV_E4M3);
    else LAUNCH(64, KV_E5M2);
  }
#undef LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}

OME_API int ome_kv_cache_write(const void* k, const void* v, int64_t kv_stride, void* k_cache, void* v_cache,
                               const int* slots, int T, int Hkv, int D, int P, int kv_fmt, float k_scale,
                               float v_scale, hipStream_t stream) {
  if (T <= 0) return 0;
  if ((D != 128 && D != 64 && D != 256) || P != 16) return -4;
  if (kv_fmt < 0 || kv_fmt > 2) return -5;
  const float ki = 1.f / k_scale, vi = 1.f / v_scale;
#define LAUNCH(DD, FF)                                                                                    \
  kv_cache_write_kernel<DD, 16, FF><<<T, 128, 0, stream>>>((const bf16*)k, (const bf16*)v, kv_stride,   \
                                                           (KVStore<FF>::T*)k_cache,                     \
                                                           (KVStore<FF>::T*)v_cache, slots, Hkv, ki, vi)
  if (D == 128) {
    if (kv_fmt == KV_BF16) LAUNCH(128, KV_BF16);
    else if (kv_fmt == KV_E4M3) LAUNCH(128, KV_E4M3);
    else LAUNCH(128, KV_E5M2);
  } else if (D == 256) {
    if (kv_fmt == KV_BF16) LAUNCH(256, KV_BF16);
    else if (kv_fmt == KV_E4M3) LAUNCH(256, KV_E4M3);
    else LAUNCH(256, KV_E5M2);
  } else {
    if (kv_fmt == KV_BF16) LAUNCH(64, KV_BF16);
    else if (kv_fmt == KV_E4M3) LAUNCH(64, KV_E4M3);
    else LAUNCH(64, KV_E5M2);
  }
#undef LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}


// ---- projection-wide q / k RMSNorm + partial rotary + paged write, any head width <= D ----
// One 256-thread workgroup per token.  q [Hq*dim] and k [Hkv*dim] are each normalised by ONE root
// mean square over the whole projection row (weights of that width; null = no norm), then the
// first rot_dim dims of every head are rotated (interleaved: dim 2i with 2i+1; else i with
// i + rot_dim/2) by the angle row cos_sin[pos] = [cos(rot_dim/2) | sin(rot_dim/2)], all in fp32
// with one rounding to bf16 at the store.  Heads are written D wide (q_out [T, Hq, D], K cache
// [page, Hkv, P, D], V cache [page, Hkv, D, P]) with zeros beyond dim / vdim.  q_scale (fp32 [Hq],
// nullable): a per-head factor on the rotated query (a temperature), applied in fp32 before the
// rounding.  v_rep > 1: v holds Hkv / v_rep heads and cache head h stores value head h / v_rep
// (several key heads attending over the same values).
template <typename T>
__global__ __launch_bounds__(256) void wide_norm_rope_cache_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride,
    const T* __restrict__ v, int64_t v_stride, const int* __restrict__ positions,
    const float* __restrict__ cos_sin, int rot_dim, int interleaved, const T* __restrict__ qn_w,
    const T* __restrict__ kn_w, float eps, T* __restrict__ q_out, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int* __restrict__ slots, int Hq, int Hkv, int dim, int vdim, int D, int P,
    const float* __restrict__ q_scale, int v_rep) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const T* qr = q + t * q_stride;
  const T* kr = k + t * k_stride;
  const T* vr = v + t * v_stride;
  const int nq = Hq * dim, nk = Hkv * dim;
  float rq = 1.f, rk = 1.f;
  if (qn_w != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nq; i += 256) ss += (float)qr[i] * (float)qr[i];
    rq = 1.f / sqrtf(block_sum<256>(ss, red) / (float)nq + eps);
  }
  if (kn_w != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x; i < nk; i += 256) ss += (float)kr[i] * (float)kr[i];
    rk = 1.f / sqrtf(block_sum<256>(ss, red) / (float)nk + eps);
  }
  const int half = rot_dim >> 1;
  const float* cs = cos_sin + (int64_t)positions[t] * rot_dim;
  const int slot = slots[t];
  const int64_t page = slot >= 0 ? slot / P : 0, off = slot >= 0 ? slot % P : 0;
  const int hp = D >> 1;   // dim pairs per (padded) head
  // q and k: one unit = one pair of dims of one head
  for (int u = threadIdx.x; u < (Hq + Hkv) * hp; u += 256) {
    const int h = u / hp, j = u - h * hp;
    const bool is_q = h < Hq;
    const int hh = is_q ? h : h - Hq;
    int d0, d1;
    if (j < half) {
      d0 = interleaved ? 2 * j : j;
      d1 = interleaved ? 2 * j + 1 : j + half;
    } else {
      d0 = rot_dim + 2 * (j - half);
      d1 = d0 + 1;
    }
    const T* src = is_q ? qr : kr;
    const T* nw = is_q ? qn_w : kn_w;
    const float rs = is_q ? rq : rk;
    float a = 0.f, b = 0.f;
    if (d0 < dim) {
      a = (float)src[hh * dim + d0];
      if (nw != nullptr) a = a * rs * (float)nw[hh * dim + d0];
    }
    if (d1 < dim) {
      b = (float)src[hh * dim + d1];
      if (nw != nullptr) b = b * rs * (float)nw[hh * dim + d1];
    }
    if (j < half) {
      const float c = cs[j], sn = cs[half + j];
      const float ra = a * c - b * sn, rb = b * c + a * sn;
      a = ra;
      b = rb;
    }
    if (is_q) {
      T* dst = q_out + (t * Hq + hh) * D;
      if (q_scale != nullptr) {
        a *= q_scale[hh];
        b *= q_scale[hh];
      }
      if (d0 < D) dst[d0] = (T)a;
      if (d1 < D) dst[d1] = (T)b;
    } else if (slot >= 0) {
      T* dst = k_cache + ((page * Hkv + hh) * P + off) * D;
      if (d0 < D) dst[d0] = (T)a;
      if (d1 < D) dst[d1] = (T)b;
    }
  }
  // v: transposed scatter [page][kh][d][off], zeros beyond vdim
  if (slot >= 0) {
    for (int i = threadIdx.x; i < Hkv * D; i += 256) {
      const int kh = i / D, d = i - kh * D;
      const float x = d < vdim ? (float)vr[(kh / v_rep) * vdim + d] : 0.f;
      v_cache[((page * Hkv + kh) * D + d) * P + off] = (T)x;
    }
  }
}

// The same op with 16-byte accesses, for the shapes real layers have: interleaved rotation (a
// pair never leaves its 8-wide vector) or half-split pairs with rot_dim % 16 == 0 (the partner is
// the vector rot_dim / 2 further or nearer, read as a second vector), dim % 8 == 0, rows and
// pointers 16-byte aligned.  A unit is one 8-dim vector of one head; pass one sums the squares from
// vector loads, pass two re-reads the (cache-hot) row, normalises, rotates in registers and stores
// one vector.
__global__ __launch_bounds__(256) void wide_norm_rope_cache_vec_kernel(
    const bf16* __restrict__ q, int64_t q_stride, const bf16* __restrict__ k, int64_t k_stride,
    const bf16* __restrict__ v, int64_t v_stride, const int* __restrict__ positions,
    const float* __restrict__ cos_sin, int rot_dim, const bf16* __restrict__ qn_w, const bf16* __restrict__ kn_w,
    float eps, bf16* __restrict__ q_out, bf16* __restrict__ k_cache, bf16* __restrict__ v_cache,
    const int* __restrict__ slots, int Hq, int Hkv, int dim, int vdim, int D, int P,
    const float* __restrict__ q_scale, int v_rep, int interleaved) {
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const bf16* qr = q + t * q_stride;
  const bf16* kr = k + t * k_stride;
  const bf16* vr = v + t * v_stride;
  const int nq = Hq * dim, nk = Hkv * dim;
  float rq = 1.f, rk = 1.f;
  if (qn_w != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x * 8; i < nq; i += 2048) {
      const bf16x8 x = ld8(qr + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)x[j] * (float)x[j];
    }
    rq = 1.f / sqrtf(block_sum<256>(ss, red) / (float)nq + eps);
  }
  if (kn_w != nullptr) {
    float ss = 0.f;
    for (int i = threadIdx.x * 8; i < nk; i += 2048) {
      const bf16x8 x = ld8(kr + i);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss += (float)x[j] * (float)x[j];
    }
    rk = 1.f / sqrtf(block_sum<256>(ss, red) / (float)nk + eps);
  }
  const int half = rot_dim >> 1;
  const float* cs = cos_sin + (int64_t)positions[t] * rot_dim;
  const int slot = slots[t];
  const int64_t page = slot >= 0 ? slot / P : 0, off = slot >= 0 ? slot % P : 0;
  const int vph = D >> 3;   // vectors per (padded) head
  for (int u = threadIdx.x; u < (Hq + Hkv) * vph; u += 256) {
    const int h = u / vph, d0 = (u - h * vph) * 8;
    const bool is_q = h < Hq;
    const int hh = is_q ? h : h - Hq;
    if (!is_q && slot < 0) continue;
    bf16x8 o = {};
    if (d0 < dim) {
      const bf16* src = (is_q ? qr : kr) + hh * dim + d0;
      const bf16* nw = is_q ? qn_w : kn_w;
      const bf16x8 x = ld8(src);
      float f[8];
      if (nw != nullptr) {
        const bf16x8 wv = ld8(nw + hh * dim + d0);
        const float rs = is_q ? rq : rk;
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = (float)x[j] * rs * (float)wv[j];
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) f[j] = (float)x[j];
      }
      if (interleaved) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int d = d0 + 2 * j;
          if (d < rot_dim) {
            const float c = cs[d >> 1], sn = cs[half + (d >> 1)];
            const float a = f[2 * j], b = f[2 * j + 1];
            f[2 * j] = a * c - b * sn;
            f[2 * j + 1] = b * c + a * sn;
          }
        }
      } else if (d0 < rot_dim) {   // half-split: dim d pairs with d + half (d < half) or d - half
        const bool lowh = d0 < half;
        const int dp = lowh ? d0 + half : d0 - half, a0 = lowh ? d0 : dp;
        const bf16x8 y = ld8(src - d0 + dp);
        float pv[8];
        if (nw != nullptr) {
          const bf16x8 wv = ld8(nw + hh * dim + dp);
          const float rs = is_q ? rq : rk;
#pragma unroll
          for (int j = 0; j < 8; ++j) pv[j] = (float)y[j] * rs * (float)wv[j];
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) pv[j] = (float)y[j];
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float c = cs[a0 + j], sn = cs[half + a0 + j];
          f[j] = lowh ? f[j] * c - pv[j] * sn : f[j] * c + pv[j] * sn;
        }
      }
      const float qs = is_q && q_scale != nullptr ? q_scale[hh] : 1.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (bf16)(f[j] * qs);
    }
    if (is_q) st8(q_out + (t * Hq + hh) * D + d0, o);
    else st8(k_cache + ((page * Hkv + hh) * P + off) * D + d0, o);
  }
  if (slot >= 0) {   // v: lanes take consecutive dims (rows 2 * P bytes apart), zeros beyond vdim
    for (int i = threadIdx.x; i < Hkv * D; i += 256) {
      const int kh = i / D, d = i - kh * D;
      v_cache[((page * Hkv + kh) * D + d) * P + off] = d < vdim ? vr[(kh / v_rep) * vdim + d] : (bf16)0.f;
    }
  }
}

OME_API int ome_wide_norm_rope_cache(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                     int64_t v_stride, const int* positions, const float* cos_sin, int rot_dim,
                                     int interleaved, const void* qn_w, const void* kn_w, float eps, void* q_out,
                                     void* k_cache, void* v_cache, const int* slots, int T, int Hq, int Hkv, int dim,
                                     int vdim, int D, int P, int f32, const float* q_scale, int v_rep,
                                     hipStream_t stream) {
  if (T <= 0) return 0;
  if (dim <= 0 || vdim <= 0 || dim > D || vdim > D || (D & 1) || rot_dim < 0 || rot_dim > dim || (rot_dim & 1))
    return -2;
  if (v_rep < 1 || Hkv % v_rep) return -2;
  if (f32) {   // fp32 model: fp32 projections, norm weights, q and cache
    wide_norm_rope_cache_kernel<float><<<T, 256, 0, stream>>>(
        (const float*)q, q_stride, (const float*)k, k_stride, (const float*)v, v_stride, positions, cos_sin, rot_dim,
        interleaved, (const float*)qn_w, (const float*)kn_w, eps, (float*)q_out, (float*)k_cache, (float*)v_cache,
        slots, Hq, Hkv, dim, vdim, D, P, q_scale, v_rep);
    OME_CHECK_LAUNCH();
    return 0;
  }
  const bool vec = (interleaved || rot_dim % 16 == 0) && dim % 8 == 0 && D % 8 == 0 && q_stride % 8 == 0 &&
                   k_stride % 8 == 0 &&
                   (uintptr_t)q % 16 == 0 && (uintptr_t)k % 16 == 0 && (uintptr_t)q_out % 16 == 0 &&
                   (uintptr_t)k_cache % 16 == 0 && (qn_w == nullptr || (uintptr_t)qn_w % 16 == 0) &&
                   (kn_w == nullptr || (uintptr_t)kn_w % 16 == 0);
  if (vec) {
    wide_norm_rope_cache_vec_kernel<<<T, 256, 0, stream>>>(
        (const bf16*)q, q_stride, (const bf16*)k, k_stride, (const bf16*)v, v_stride, positions, cos_sin, rot_dim,
        (const bf16*)qn_w, (const bf16*)kn_w, eps, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, slots, Hq, Hkv, dim,
        vdim, D, P, q_scale, v_rep, interleaved);
    OME_CHECK_LAUNCH();
    return 0;
  }
  wide_norm_rope_cache_kernel<bf16><<<T, 256, 0, stream>>>(
      (const bf16*)q, q_stride, (const bf16*)k, k_stride, (const bf16*)v, v_stride, positions, cos_sin, rot_dim,
      interleaved, (const bf16*)qn_w, (const bf16*)kn_w, eps, (bf16*)q_out, (bf16*)k_cache, (bf16*)v_cache, slots,
      Hq, Hkv, dim, vdim, D, P, q_scale, v_rep);
  OME_CHECK_LAUNCH();
  return 0;
}

// ------------------------------------------------------------------------------------------
// Attention input with short causal convolutions: q, k, v (row-strided views of one projection)
// each pass a depthwise convolution over time (K taps per channel, no bias, no activation), then
// q and k get the rotary embedding on the first rot_dim dims of every head (interleaved pairs
// 2i / 2i+1, or halves i / i + rot_dim/2; angles from the fp32 cos | sin table row of the token's
// position) and, AFTER the rotation, each head is divided by its root mean square over `dim`
// (unit_norm; no weight).  q goes to q_out [T, Hq, D], k / v into the paged cache (K [pages, Hkv,
// P, D], V [pages, Hkv, D, P]); head tails beyond dim / vdim are written as zeros (q, k) or left
// as the cache's zeros (v).  Convolution sum, angles, rotation and norm are fp32; one rounding at
// the store.
//
// The last K-1 projected rows of every sequence live in `tail` [slots, K-1, C] (C = all q, k, v
// channels; row j = input at time -(K-1) + j of the next step).  Time is tiled: one workgroup =
// (head of q / k / v, sequence, tile of CR_TILE rows); a wave owns a row at a time, lanes own the
// head's channels.  Only a sequence's first tile touches the tail: it reads the old rows into LDS
// and then writes the new ones from the step's last rows (or the shifted old rows of a step
// shorter than K-1), so tiles never race.  K == 0: no convolution (and no tail).
// ------------------------------------------------------------------------------------------
namespace {
constexpr int CR_TILE = 32;
constexpr int CR_MAXS = 1024;   // sequence starts staged in LDS (more: read from global memory)

template <typename T>
__global__ __launch_bounds__(256) void conv_rope_cache_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ wq, const T* __restrict__ wk, const T* __restrict__ wv, int K,
    T* __restrict__ tail, const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ reset,
    const int* __restrict__ positions, const float* __restrict__ cos_sin, int rot_dim, int interleaved,
    int unit_norm, float eps, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
    const int* __restrict__ slots, int Hq, int Hkv, int dim, int vdim, int D, int P, int S) {
  extern __shared__ float sm[];   // [CR_TILE + K - 1][d] input rows, then [K][d] taps
  const int hh = blockIdx.x;
  // blockIdx.y counts the tiles of all sequences in turn (the grid is the upper bound T / CR_TILE + S);
  // the sequence starts are staged in LDS so that the walk is not a chain of global loads
  __shared__ int s_cu[CR_MAXS + 1];
  const bool staged = S <= CR_MAXS;
  if (staged) {
    for (int i = threadIdx.x; i <= S; i += 256) s_cu[i] = cu[i];
    __syncthreads();
  }
  const int* cus = staged ? s_cu : cu;
  int s = 0, z = blockIdx.y;
  for (; s < S; ++s) {
    const int n = (cus[s + 1] - cus[s] + CR_TILE - 1) / CR_TILE;
    if (z < n) break;
    z -= n;
  }
  if (s >= S) return;
  const int r0 = cus[s], r1 = cus[s + 1];
  const int a = r0 + z * CR_TILE;
  const int e = min(a + CR_TILE, r1);
  const int kind = hh < Hq ? 0 : (hh < Hq + Hkv ? 1 : 2);
  const int head = kind == 0 ? hh : (kind == 1 ? hh - Hq : hh - Hq - Hkv);
  const int d = kind == 2 ? vdim : dim;
  const T* src = kind == 0 ? q : (kind == 1 ? k : v);
  const int64_t sstride = kind == 0 ? q_stride : (kind == 1 ? k_stride : v_stride);
  const T* wt = kind == 0 ? wq : (kind == 1 ? wk : wv);
  const int C = Hq * dim + Hkv * dim + Hkv * vdim;
  const int c0 = kind == 0 ? head * dim : (kind == 1 ? Hq * dim + head * dim : (Hq + Hkv) * dim + head * vdim);
  const int KT = K > 0 ? K - 1 : 0;
  float* rows = sm;
  float* taps = sm + (CR_TILE + KT) * d;
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63;
  // A global load costs a round trip of a microsecond under load, so the kernel is arranged as a few
  // rounds of independent loads: (1) the rows' positions / cache slots (lane i of a wave holds row
  // wave + 4 i of the tile) together with the sequence's slot and the input rows and taps, (2) the
  // rows' cos / sin, all asked for before the row loop, which then runs out of LDS and registers.
  constexpr int RPW = CR_TILE / 4;   // rows per wave
  int my_pos = 0, my_slot = -1;
  if (lane < RPW && a + wave + 4 * lane < e) {
    my_pos = positions[a + wave + 4 * lane];
    my_slot = slots[a + wave + 4 * lane];
  }
  T* tl = KT > 0 ? tail + (int64_t)slot[s] * KT * C + c0 : nullptr;
  const bool fresh = reset[s] != 0;
  for (int i = tid; i < K * d; i += 256) taps[i] = (float)wt[(int64_t)(head * d + i % d) * K + i / d];   // [j][c]
  // input rows a - KT .. e - 1 of the sequence (before r0: the old tail, or zeros)
  const bool vec = sizeof(T) == 2 && (d & 7) == 0 && (sstride & 7) == 0 && (C & 7) == 0 &&
                   ((uintptr_t)src & 15) == 0 && (tl == nullptr || ((uintptr_t)tl & 15) == 0);
  if (vec) {
    const int cpr = d >> 3;   // 16-byte pieces per row
    const int total = (e - a + KT) * cpr;
    for (int base = 0; base < total; base += 256 * 4) {
      bf16x8 x[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {   // all loads of the round first
        const int i = base + tid + 256 * u;
        x[u] = bf16x8{};
        if (i < total) {
          const int rr = i / cpr, c = (i - rr * cpr) << 3;
          const int r = a - KT + rr;
          if (r >= r0) x[u] = ld8((const bf16*)src + (int64_t)r * sstride + head * d + c);
          else if (!fresh) x[u] = ld8((const bf16*)tl + (int64_t)(KT + (r - r0)) * C + c);
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + tid + 256 * u;
        if (i < total) {
          const int rr = i / cpr, c = (i - rr * cpr) << 3;
#pragma unroll
          for (int j = 0; j < 8; ++j) rows[rr * d + c + j] = (float)x[u][j];
        }
      }
    }
  } else {
    for (int i = tid; i < (e - a + KT) * d; i += 256) {
      const int rr = i / d, c = i - rr * d;
      const int r = a - KT + rr;
      float x;
      if (r >= r0) x = (float)src[(int64_t)r * sstride + head * d + c];
      else x = fresh ? 0.f : (float)tl[(int64_t)(KT + (r - r0)) * C + c];
      rows[rr * d + c] = x;
    }
  }
  // cos / sin of this wave's rows: lane -> pairs 2 lane (, 128 + 2 lane) -> table columns lane (, 64 + lane)
  const int half = rot_dim >> 1;
  float co[RPW][2], si[RPW][2];
  if (kind != 2 && rot_dim > 0 && interleaved) {
#pragma unroll
    for (int it = 0; it < RPW; ++it) {
      const int pos = __shfl(my_pos, it);
      const float* cs = cos_sin + (int64_t)pos * rot_dim;
#pragma unroll
      for (int pr = 0; pr < 2; ++pr) {
        const int ci = 64 * pr + lane;   // pair index
        const bool on = 2 * ci < rot_dim && a + wave + 4 * it < e;
        co[it][pr] = on ? cs[ci] : 1.f;
        si[it][pr] = on ? cs[half + ci] : 0.f;
      }
    }
  }
  __syncthreads();
  if (z == 0 && KT > 0) {   // new tail: inputs L - KT .. L - 1 of the step; negative = old tail rows
    const int L = r1 - r0;
    for (int i = tid; i < KT * d; i += 256) {
      const int j = i / d, c = i - j * d;
      const int t = L - KT + j;
      tl[(int64_t)j * C + c] = t >= 0 ? src[(int64_t)(r0 + t) * sstride + head * d + c] : (T)rows[(KT + t) * d + c];
    }
  }
  // a lane owns two pairs of neighbouring channels: register u <-> channel (u >> 1) * 128 + 2 lane + (u & 1)
  // (d <= 256), so an interleaved rotary pair sits in one lane and stores are 4 bytes wide
#pragma unroll
  for (int it = 0; it < RPW; ++it) {
    const int rr = wave + 4 * it;   // output row rr reads input rows rr .. rr + KT
    const int r = a + rr;
    const int slot_t = __shfl(my_slot, it);
    const int pos = __shfl(my_pos, it);
    if (r >= e) continue;
    float y[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int c = (u >> 1) * 128 + 2 * lane + (u & 1);
      float acc = 0.f;
      if (c < d) {
        if (K > 0)
          for (int j = 0; j < K; ++j) acc += taps[j * d + c] * rows[(rr + j) * d + c];
        else
          acc = rows[rr * d + c];
      }
      y[u] = acc;
    }
    if (kind == 2) {
      if (slot_t >= 0) {
        T* vc = v_cache + (((int64_t)(slot_t / P) * Hkv + head) * D) * P + slot_t % P;
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = (u >> 1) * 128 + 2 * lane + (u & 1);
          if (c < d) vc[(int64_t)c * P] = (T)y[u];
        }
      }
      continue;
    }
    if (rot_dim > 0) {
      if (interleaved) {
#pragma unroll
        for (int u = 0; u < 4; u += 2) {
          const float ev = y[u], od = y[u + 1];
          y[u] = ev * co[it][u >> 1] - od * si[it][u >> 1];
          y[u + 1] = od * co[it][u >> 1] + ev * si[it][u >> 1];
        }
      } else {   // channel i pairs with i + half: the partner pc sits in lane (pc & 127) >> 1, register
        // (pc >> 7) * 2 + (pc & 1)
        const float* cs = cos_sin + (int64_t)pos * rot_dim;
        float other[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = (u >> 1) * 128 + 2 * lane + (u & 1);
          const int pc = c < half ? c + half : c - half;
          const int pl = (pc & 127) >> 1, pr = ((pc >> 7) << 1) | (pc & 1);
          float o = 0.f;
#pragma unroll
          for (int u2 = 0; u2 < 4; ++u2) {
            const float cand = __shfl(y[u2], pl);
            if (pr == u2) o = cand;
          }
          other[u] = o;
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int c = (u >> 1) * 128 + 2 * lane + (u & 1);
          if (c < rot_dim) {
            const int i = c < half ? c : c - half;
            const float cc = cs[i], ss = cs[half + i];
            y[u] = c < half ? y[u] * cc - other[u] * ss : y[u] * cc + other[u] * ss;
          }
        }
      }
    }
    if (unit_norm) {
      float ss = 0.f;
#pragma unroll
      for (int u = 0; u < 4; ++u) ss += ((u >> 1) * 128 + 2 * lane + (u & 1) < d) ? y[u] * y[u] : 0.f;
      const float rs = 1.f / sqrtf(wave_sum(ss) / (float)d + eps);
#pragma unroll
      for (int u = 0; u < 4; ++u) y[u] *= rs;
    }
    T* dst;
    if (kind == 0) dst = q_out + ((int64_t)r * Hq + head) * D;
    else dst = slot_t >= 0 ? k_cache + (((int64_t)(slot_t / P) * Hkv + head) * P + slot_t % P) * D : nullptr;
    if (dst != nullptr) {
#pragma unroll
      for (int u = 0; u < 4; u += 2) {
        const int c = (u >> 1) * 128 + 2 * lane;      // D is even, so a pair is inside or outside together
        if (c < D) {
          const T lo_v = c < d ? (T)y[u] : (T)0.f, hi_v = c + 1 < d ? (T)y[u + 1] : (T)0.f;
          if constexpr (sizeof(T) == 2) {
            *reinterpret_cast<bf16x2*>(dst + c) = bf16x2{(bf16)lo_v, (bf16)hi_v};
          } else {
            dst[c] = lo_v;
            dst[c + 1] = hi_v;
          }
        }
      }
    }
  }
}
}  // namespace

// ------------------------------------------------------------------------------------------
// The same step for the common shapes (head widths in multiples of 8, up to CV_MAXK taps,
// interleaved rotary pairs, 16-byte aligned rows), without LDS and without barriers: one item =
// (row, head of q / k / v), a lane owns 8 neighbouring channels (D / 8 lanes per item), reads its K
// input vectors straight from the projection rows (L1 / L2 keep the K-fold reuse) or, for rows
// before the step's first, from the sequence's tail, and writes 16-byte vectors.  Per row the
// caller gives the sequence's first row of the step (row_start) and its state slot (row_slot,
// bit 30 set: the sequence starts here, its tail counts as zeros).  The tails are rewritten by
// conv_tail_kernel AFTER this kernel (stream order), one thread per (sequence, channel), which
// reads a channel's old tail before it writes the new one.
// ------------------------------------------------------------------------------------------
namespace {
constexpr int CV_MAXK = 6;

template <typename T>
__device__ __forceinline__ void cv_ld8(const T* p, float (&f)[8]) {
  if constexpr (sizeof(T) == 2) {
    const bf16x8 t = ld8((const bf16*)p);
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = (float)t[j];
  } else {
    const f32x4 a = *reinterpret_cast<const f32x4*>(p), b = *reinterpret_cast<const f32x4*>(p + 4);
    f[0] = a[0]; f[1] = a[1]; f[2] = a[2]; f[3] = a[3];
    f[4] = b[0]; f[5] = b[1]; f[6] = b[2]; f[7] = b[3];
  }
}
template <typename T>
__device__ __forceinline__ void cv_st8(T* p, const float (&f)[8]) {
  if constexpr (sizeof(T) == 2) {
    bf16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (bf16)f[j];
    st8((bf16*)p, o);
  } else {
    *reinterpret_cast<f32x4*>(p) = f32x4{f[0], f[1], f[2], f[3]};
    *reinterpret_cast<f32x4*>(p + 4) = f32x4{f[4], f[5], f[6], f[7]};
  }
}

// K = taps (0: no convolution); GS = lanes per item = D / 8
template <typename T, int K, int GS>
__global__ __launch_bounds__(256) void conv_rope_cache_vec_kernel(
    const T* __restrict__ q, int64_t q_stride, const T* __restrict__ k, int64_t k_stride, const T* __restrict__ v,
    int64_t v_stride, const T* __restrict__ wq, const T* __restrict__ wk, const T* __restrict__ wv,
    const T* __restrict__ tail, const int* __restrict__ row_start, const int* __restrict__ row_slot,
    const int* __restrict__ positions, const float* __restrict__ cos_sin, int rot_dim, int unit_norm, float eps,
    T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ slots, int Tn,
    int Hq, int Hkv, int dim, int vdim, int P) {
  constexpr int D = GS * 8, KT = K > 0 ? K - 1 : 0, KK = K > 0 ? K : 1;
  const int Ht = Hq + 2 * Hkv;
  const int64_t item = (int64_t)blockIdx.x * (256 / GS) + threadIdx.x / GS;
  const int l = threadIdx.x % GS;
  const bool live = item < (int64_t)Tn * Ht;
  // items go row by row within a head: the items of a wave share the head's taps and overlap in the
  // input rows they read (cache hits), and neighbouring lanes' rows are neighbours
  const int hh = live ? (int)(item / Tn) : 0;
  const int t = live ? (int)(item - (int64_t)hh * Tn) : 0;
  const int kind = hh < Hq ? 0 : (hh < Hq + Hkv ? 1 : 2);
  const int head = kind == 0 ? hh : (kind == 1 ? hh - Hq : hh - Hq - Hkv);
  const int d = kind == 2 ? vdim : dim;
  const T* src = kind == 0 ? q : (kind == 1 ? k : v);
  const int64_t sstride = kind == 0 ? q_stride : (kind == 1 ? k_stride : v_stride);
  const T* wt = kind == 0 ? wq : (kind == 1 ? wk : wv);
  const int C = Hq * dim + Hkv * dim + Hkv * vdim;
  const int c0 = kind == 0 ? head * dim : (kind == 1 ? Hq * dim + head * dim : (Hq + Hkv) * dim + head * vdim);
  const int c8 = 8 * l;
  const bool on = live && c8 < d;       // (d is a multiple of 8: a lane's channels are all inside or all outside)
  // round 1: the row's sequence, position and cache slot
  const int r0 = row_start[t], rs = row_slot[t], pos = positions[t], slot_t = slots[t];
  const bool fresh = (rs >> 30) & 1;
  const int st = rs & 0x3fffffff;
  // round 2: inputs and taps
  float x[KK][8], w[8 * KK];
#pragma unroll
  for (int j = 0; j < KK; ++j) {
    const int r = t - KT + j;
#pragma unroll
    for (int e = 0; e < 8; ++e) x[j][e] = 0.f;
    if (on) {
      if (r >= r0) cv_ld8<T>(src + (int64_t)r * sstride + head * d + c8, x[j]);
      else if (!fresh) cv_ld8<T>(tail + ((int64_t)st * KT + (KT + r - r0)) * C + c0 + c8, x[j]);
    }
  }
  float y[8];
  if constexpr (K > 0) {
    if (on) {   // this lane's taps are contiguous: w[e * K + j]
#pragma unroll
      for (int m = 0; m < K; ++m) {
        float tmp[8];
        cv_ld8<T>(wt + (int64_t)(head * d + c8) * K + 8 * m, tmp);
#pragma unroll
        for (int e = 0; e < 8; ++e) w[8 * m + e] = tmp[e];
      }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      float acc = 0.f;
#pragma unroll
      for (int j = 0; j < K; ++j) acc += w[e * K + j] * x[j][e];
      y[e] = on ? acc : 0.f;
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) y[e] = x[0][e];
  }
  if (kind == 2) {
    if (on && slot_t >= 0) {
      T* vc = v_cache + (((int64_t)(slot_t / P) * Hkv + head) * D + c8) * P + slot_t % P;
#pragma unroll
      for (int e = 0; e < 8; ++e) vc[(int64_t)e * P] = (T)y[e];
    }
  }
  // (q / k from here; lanes of value items only take part in the shuffles)
  if (kind != 2 && on && rot_dim > 0) {
    const float* cs = cos_sin + (int64_t)pos * rot_dim;
    const int half = rot_dim >> 1;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      const int c = c8 + e;
      if (c < rot_dim) {
        const float co = cs[c >> 1], si = cs[half + (c >> 1)];
        const float ev = y[e], od = y[e + 1];
        y[e] = ev * co - od * si;
        y[e + 1] = od * co + ev * si;
      }
    }
  }
  if (unit_norm) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += y[e] * y[e];
#pragma unroll
    for (int o = GS / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
    const float rsq = 1.f / sqrtf(ss / (float)d + eps);
    if (kind != 2) {
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] *= rsq;
    }
  }
  if (live && kind != 2) {   // every lane of the item writes its 16 bytes: zeros beyond the head's width
    T* dst;
    if (kind == 0) dst = q_out + ((int64_t)t * Hq + head) * D;
    else dst = slot_t >= 0 ? k_cache + (((int64_t)(slot_t / P) * Hkv + head) * P + slot_t % P) * D : nullptr;
    if (dst != nullptr) cv_st8<T>(dst + c8, y);
  }
}

// new tail of every sequence: inputs L - KT .. L - 1 of the step (negative: the old tail, shifted)
template <typename T>
__global__ __launch_bounds__(256) void conv_tail_kernel(const T* __restrict__ q, int64_t q_stride,
                                                        const T* __restrict__ k, int64_t k_stride,
                                                        const T* __restrict__ v, int64_t v_stride,
                                                        T* __restrict__ tail, const int* __restrict__ cu,
                                                        const int* __restrict__ slot, const int* __restrict__ reset,
                                                        int KT, int nq, int nk, int C) {
  const int c = blockIdx.x * 256 + threadIdx.x, s = blockIdx.y;
  if (c >= C) return;
  const int r0 = cu[s], L = cu[s + 1] - r0;
  if (L <= 0) return;
  const T* src = c < nq ? q + c : (c < nq + nk ? k + (c - nq) : v + (c - nq - nk));
  const int64_t stride = c < nq ? q_stride : (c < nq + nk ? k_stride : v_stride);
  T* tl = tail + (int64_t)slot[s] * KT * C + c;
  const bool fresh = reset[s] != 0;
  T val[32];
  for (int j = 0; j < KT; ++j) {
    const int t = L - KT + j;
    val[j] = t >= 0 ? src[(int64_t)(r0 + t) * stride] : (fresh ? (T)0.f : tl[(int64_t)(j + L) * C]);
  }
  for (int j = 0; j < KT; ++j) tl[(int64_t)j * C] = val[j];
}
}  // namespace

// Fast path of ome_conv_rope_cache (see conv_rope_cache_vec_kernel).  Returns -9 when the shapes
// are not the ones it is built for: the caller then takes the general kernel.
OME_API int ome_conv_rope_cache_vec(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                    int64_t v_stride, const void* wq, const void* wk, const void* wv, int K,
                                    void* tail, const int* cu, const int* slot, const int* reset, int S,
                                    const int* row_start, const int* row_slot, const int* positions,
                                    const float* cos_sin, int rot_dim, int unit_norm, float eps, void* q_out,
                                    void* k_cache, void* v_cache, const int* slots, int T, int Hq, int Hkv, int dim,
                                    int vdim, int D, int P, int f32, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  const int esz = f32 ? 4 : 2;
  auto al = [&](const void* p, int64_t stride) { return (((uintptr_t)p | (uintptr_t)(stride * esz)) & 15) == 0; };
  if (K < 0 || K > CV_MAXK || dim % 8 || vdim % 8 || dim > D || vdim > D || (D != 64 && D != 128 && D != 256) ||
      (rot_dim & 1) || rot_dim > dim || !al(q, q_stride) || !al(k, k_stride) || !al(v, v_stride) || !al(wq, 0) ||
      !al(wk, 0) || !al(wv, 0) || !al(tail, 0) || !al(q_out, 0) || !al(k_cache, 0) ||
      (((int64_t)(Hq + Hkv) * dim + (int64_t)Hkv * vdim) * esz) % 16)
    return -9;
  if (K > 1 && tail == nullptr) return -2;
  const int gs = D / 8;
  const int64_t items = (int64_t)T * (Hq + 2 * Hkv);
  const unsigned grid = (unsigned)((items + 256 / gs - 1) / (256 / gs));
#define CV_ARGS(TT)                                                                                                 \
  (const TT*)q, q_stride, (const TT*)k, k_stride, (const TT*)v, v_stride, (const TT*)wq, (const TT*)wk,            \
      (const TT*)wv, (const TT*)tail, row_start, row_slot, positions, cos_sin, rot_dim, unit_norm, eps, (TT*)q_out, \
      (TT*)k_cache, (TT*)v_cache, slots, T, Hq, Hkv, dim, vdim, P
#define CV_GS(TT, KK)                                                                                   \
  do {                                                                                                  \
    if (gs == 8) conv_rope_cache_vec_kernel<TT, KK, 8><<<grid, 256, 0, stream>>>(CV_ARGS(TT));          \
    else if (gs == 16) conv_rope_cache_vec_kernel<TT, KK, 16><<<grid, 256, 0, stream>>>(CV_ARGS(TT));   \
    else conv_rope_cache_vec_kernel<TT, KK, 32><<<grid, 256, 0, stream>>>(CV_ARGS(TT));                 \
  } while (0)
#define CV_K(TT)                     \
  switch (K) {                       \
    case 0: CV_GS(TT, 0); break;     \
    case 1: CV_GS(TT, 1); break;     \
    case 2: CV_GS(TT, 2); break;     \
    case 3: CV_GS(TT, 3); break;     \
    case 4: CV_GS(TT, 4); break;     \
    case 5: CV_GS(TT, 5); break;     \
    default: CV_GS(TT, 6); break;    \
  }
  if (f32) { CV_K(float) } else { CV_K(bf16) }
#undef CV_K
#undef CV_GS
#undef CV_ARGS
  OME_CHECK_LAUNCH();
  if (K > 1) {
    const int C = (Hq + Hkv) * dim + Hkv * vdim;
    const dim3 g2((C + 255) / 256, S);
    if (S > 65535) return -3;
    if (f32)
      conv_tail_kernel<float><<<g2, 256, 0, stream>>>((const float*)q, q_stride, (const float*)k, k_stride,
                                                      (const float*)v, v_stride, (float*)tail, cu, slot, reset, K - 1,
                                                      Hq * dim, Hkv * dim, C);
    else
      conv_tail_kernel<bf16><<<g2, 256, 0, stream>>>((const bf16*)q, q_stride, (const bf16*)k, k_stride,
                                                     (const bf16*)v, v_stride, (bf16*)tail, cu, slot, reset, K - 1,
                                                     Hq * dim, Hkv * dim, C);
    OME_CHECK_LAUNCH();
  }
  return 0;
}

OME_API int ome_conv_rope_cache(const void* q, int64_t q_stride, const void* k, int64_t k_stride, const void* v,
                                int64_t v_stride, const void* wq, const void* wk, const void* wv, int K, void* tail,
                                const int* cu, const int* slot, const int* reset, int S, const int* positions,
                                const float* cos_sin, int rot_dim, int interleaved, int unit_norm, float eps,
                                void* q_out, void* k_cache, void* v_cache, const int* slots, int T, int Hq, int Hkv,
                                int dim, int vdim, int D, int P, int f32, hipStream_t stream) {
  if (T <= 0 || S <= 0) return 0;
  if (dim <= 0 || vdim <= 0 || dim > D || vdim > D || D > 256 || K < 0 || K > 33 || rot_dim > dim || (rot_dim & 1))
    return -2;
  if (K > 0 && (wq == nullptr || wk == nullptr || wv == nullptr || (K > 1 && tail == nullptr))) return -2;
  const int tiles = (T + CR_TILE - 1) / CR_TILE + S;
  if (tiles > 65535) return -3;
  const int dmax = dim > vdim ? dim : vdim;
  const size_t lds = (size_t)((CR_TILE + (K > 0 ? K - 1 : 0)) * dmax + K * dmax) * sizeof(float);
  if (lds > 150 * 1024) return -3;   // (the staged sequence starts take 4 KB of static LDS beside it)
  dim3 grid(Hq + 2 * Hkv, tiles);
#define CRC_LAUNCH(TT)                                                                                              \
  do {                                                                                                              \
    static bool big_ = false; /* once: allow the largest dynamic LDS block */                                       \
    if (lds > 64 * 1024 && !big_) {                                                                                \
      hipError_t e_ = hipFuncSetAttribute((const void*)conv_rope_cache_kernel<TT>,                                                \
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024);                \
      if (e_ != hipSuccess) return (int)e_;                                                                        \
      big_ = true;                                                                                                 \
    }                                                                                                              \
    conv_rope_cache_kernel<TT><<<grid, 256, lds, stream>>>(                                                         \
        (const TT*)q, q_stride, (const TT*)k, k_stride, (const TT*)v, v_stride, (const TT*)wq, (const TT*)wk,       \
        (const TT*)wv, K, (TT*)tail, cu, slot, reset, positions, cos_sin, rot_dim, interleaved, unit_norm, eps,     \
        (TT*)q_out, (TT*)k_cache, (TT*)v_cache, slots, Hq, Hkv, dim, vdim, D, P, S);                                \
  } while (0)
  if (f32) CRC_LAUNCH(float);
  else CRC_LAUNCH(bf16);
#undef CRC_LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}
