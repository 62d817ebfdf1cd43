// RMSNorm and fused residual-add + RMSNorm (kernel K1 of SURVEY.md §2.9).
//
// One workgroup per token row; each lane holds its slice of the row in registers as
// 16-byte bf16x8 vectors (vectorised per Guideline 13), so the row is read once and
// written once: the op is purely HBM-bound.
#include "common.h"

template <int NT, int CHUNKS>
__global__ __launch_bounds__(NT) void rmsnorm_kernel(const bf16* __restrict__ x, int64_t x_stride,
                                                     const bf16* __restrict__ w, bf16* __restrict__ out,
                                                     int64_t out_stride, int H, float eps) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  const bf16* xr = x + row * x_stride;
  bf16* orow = out + row * out_stride;
  const int nvec = H >> 3;
  bf16x8 v[CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
      v[c] = ld8(xr + i * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        float f = (float)v[c][j];
        ss += f * f;
      }
    }
  }
  bf16x8 wv[CHUNKS];  // issue the weight loads before the reduction's barrier
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) wv[c] = ld8(w + i * 8);
  }
  ss = block_sum<NT>(ss, red);
  const float rs = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
      bf16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (bf16)((float)v[c][j] * rs * (float)wv[c][j]);
      st8(orow + i * 8, o);
    }
  }
}

// residual <- x + residual ; x <- rmsnorm(residual) * w      (in place, vLLM/SGLang semantics)
template <int NT, int CHUNKS>
__global__ __launch_bounds__(NT) void fused_add_rmsnorm_kernel(bf16* __restrict__ x, int64_t x_stride,
                                                               bf16* __restrict__ res, int64_t res_stride,
                                                               const bf16* __restrict__ w, int H,
                                                               float eps) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  bf16* xr = x + row * x_stride;
  bf16* rr = res + row * res_stride;
  const int nvec = H >> 3;
  bf16x8 v[CHUNKS];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
      bf16x8 a = ld8(xr + i * 8), b = ld8(rr + i * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        // round the sum to bf16 first: the residual stream is stored in bf16
        bf16 s = (bf16)((float)a[j] + (float)b[j]);
        v[c][j] = s;
        float f = (float)s;
        ss += f * f;
      }
      st8(rr + i * 8, v[c]);
    }
  }
  bf16x8 wv[CHUNKS];  // issue the weight loads before the reduction's barrier
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) wv[c] = ld8(w + i * 8);
  }
  ss = block_sum<NT>(ss, red);
  const float rs = rsqrtf(ss / (float)H + eps);
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
      bf16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (bf16)((float)v[c][j] * rs * (float)wv[c][j]);
      st8(xr + i * 8, o);
    }
  }
}

// LayerNorm with bias (Starcoder2, GPT-NeoX): out = (x - mean) * rstd * w + b; with ``res`` set the
// residual add is fused in front (res <- x + res, normalise res, write x), like fused_add_rmsnorm.
template <int NT, int CHUNKS, bool ADD>
__global__ __launch_bounds__(NT) void layernorm_kernel(bf16* __restrict__ x, int64_t x_stride,
                                                       bf16* __restrict__ res, int64_t res_stride,
                                                       const bf16* __restrict__ w, const bf16* __restrict__ b,
                                                       bf16* __restrict__ out, int64_t out_stride, int H, float eps) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  bf16* xr = x + row * x_stride;
  const int nvec = H >> 3;
  bf16x8 v[CHUNKS];
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
      v[c] = ld8(xr + i * 8);
      if constexpr (ADD) {
        bf16* rr = res + row * res_stride;
        const bf16x8 r = ld8(rr + i * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) v[c][j] = (bf16)((float)v[c][j] + (float)r[j]);
        st8(rr + i * 8, v[c]);
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) s += (float)v[c][j];
    }
  }
  const float mean = block_sum<NT>(s, red) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float d = (float)v[c][j] - mean;
        ss += d * d;
      }
    }
  }
  const float rstd = rsqrtf(block_sum<NT>(ss, red) / (float)H + eps);
  bf16* orow = ADD ? xr : out + row * out_stride;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int i = threadIdx.x + c * NT;
    if (i < nvec) {
      const bf16x8 wv = ld8(w + i * 8);
      bf16x8 bv = {};
      if (b != nullptr) bv = ld8(b + i * 8);
      bf16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = (bf16)(((float)v[c][j] - mean) * rstd * (float)wv[j] + (float)bv[j]);
      st8(orow + i * 8, o);
    }
  }
}

#define DISPATCH_CHUNKS(H, NT, ...)                         \
  do {                                                      \
    const int _c = ((H) / 8 + (NT)-1) / (NT);               \
    if (_c <= 1) { constexpr int CH = 1; __VA_ARGS__; }     \
    else if (_c <= 2) { constexpr int CH = 2; __VA_ARGS__; } \
    else if (_c <= 4) { constexpr int CH = 4; __VA_ARGS__; } \
    else if (_c <= 8) { constexpr int CH = 8; __VA_ARGS__; } \
    else return -1;                                         \
  } while (0)

OME_API int ome_rmsnorm(const void* x, int64_t x_stride, const void* w, void* out, int64_t out_stride,
                        int rows, int H, float eps, hipStream_t stream) {
  if (H % 8 != 0 || rows <= 0) return rows == 0 ? 0 : -2;
  // Small batches (decode) use 128-thread blocks to keep more lanes' loads in flight per CU.
  if (rows < 512) {
    DISPATCH_CHUNKS(H, 128, (rmsnorm_kernel<128, CH><<<rows, 128, 0, stream>>>(
                                (const bf16*)x, x_stride, (const bf16*)w, (bf16*)out, out_stride, H, eps)));
  } else {
    DISPATCH_CHUNKS(H, 256, (rmsnorm_kernel<256, CH><<<rows, 256, 0, stream>>>(
                                (const bf16*)x, x_stride, (const bf16*)w, (bf16*)out, out_stride, H, eps)));
  }
  OME_CHECK_LAUNCH();
  return 0;
}

static int g_norm_threads = 0;  // 0 = measured default; 128 / 256 / 512 for experiments
OME_API int ome_norm_set_threads(int nt) {
  if (nt != 0 && nt != 128 && nt != 256 && nt != 512) return -1;
  g_norm_threads = nt;
  return 0;
}

OME_API int ome_fused_add_rmsnorm(void* x, int64_t x_stride, void* res, int64_t res_stride, const void* w,
                                  int rows, int H, float eps, hipStream_t stream) {
  if (H % 8 != 0 || rows <= 0) return rows == 0 ? 0 : -2;
  if (g_norm_threads == 512) {
    DISPATCH_CHUNKS(H, 512, (fused_add_rmsnorm_kernel<512, CH><<<rows, 512, 0, stream>>>(
                                (bf16*)x, x_stride, (bf16*)res, res_stride, (const bf16*)w, H, eps)));
  } else if (g_norm_threads == 256) {
    DISPATCH_CHUNKS(H, 256, (fused_add_rmsnorm_kernel<256, CH><<<rows, 256, 0, stream>>>(
                                (bf16*)x, x_stride, (bf16*)res, res_stride, (const bf16*)w, H, eps)));
  } else if (g_norm_threads == 128) {
    DISPATCH_CHUNKS(H, 128, (fused_add_rmsnorm_kernel<128, CH><<<rows, 128, 0, stream>>>(
                                (bf16*)x, x_stride, (bf16*)res, res_stride, (const bf16*)w, H, eps)));
  } else if (rows < 512) {
    // decode batches: 8 waves per row (3.05 vs 4.15 us for 128 threads at 256 x 4096,
    // profiles/r03_small_kernels.txt)
    DISPATCH_CHUNKS(H, 512, (fused_add_rmsnorm_kernel<512, CH><<<rows, 512, 0, stream>>>(
                                (bf16*)x, x_stride, (bf16*)res, res_stride, (const bf16*)w, H, eps)));
  } else {
    DISPATCH_CHUNKS(H, 256, (fused_add_rmsnorm_kernel<256, CH><<<rows, 256, 0, stream>>>(
                                (bf16*)x, x_stride, (bf16*)res, res_stride, (const bf16*)w, H, eps)));
  }
  OME_CHECK_LAUNCH();
  return 0;
}

// res == nullptr: out = LN(x); else res <- x + res, x <- LN(res) (out unused)
OME_API int ome_layernorm(void* x, int64_t x_stride, void* res, int64_t res_stride, const void* w, const void* b,
                          void* out, int64_t out_stride, int rows, int H, float eps, hipStream_t stream) {
  if (H % 8 != 0 || rows <= 0) return rows == 0 ? 0 : -2;
  if (res != nullptr) {
    DISPATCH_CHUNKS(H, 256, (layernorm_kernel<256, CH, true><<<rows, 256, 0, stream>>>(
                                (bf16*)x, x_stride, (bf16*)res, res_stride, (const bf16*)w, (const bf16*)b,
                                nullptr, 0, H, eps)));
  } else {
    DISPATCH_CHUNKS(H, 256, (layernorm_kernel<256, CH, false><<<rows, 256, 0, stream>>>(
                                (bf16*)x, x_stride, nullptr, 0, (const bf16*)w, (const bf16*)b, (bf16*)out,
                                out_stride, H, eps)));
  }
  OME_CHECK_LAUNCH();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Per-head RMSNorm + complex-pair RoPE + row scatter (Qwen-Image MMDiT q / k; v with no norm and
// no rotation): one wave per (row, head).  x row r, head h = x[r * xs + h * HD .. +HD); w [HD] (null:
// no norm); cs [T][HD/2][2] fp32 (cos, sin) (null: no rotation); the result goes to row
// dst[r] (null: r) of out (row stride os) -- the joint [text; image] sequence is assembled by
// the writes themselves, no gather pass.  Rounding as the eager path: normed value rounded to
// bf16 before the fp32 rotation.
template <int HD>
__global__ __launch_bounds__(256) void qk_norm_rope_kernel(const bf16* __restrict__ x, int64_t xs,
                                                           const bf16* __restrict__ w, const float* __restrict__ cs,
                                                           int T, int H, float eps, bf16* __restrict__ out,
                                                           int64_t os, const int* __restrict__ dst) {
  constexpr int NP = HD / 2, PPL = (NP + 63) / 64;   // complex pairs, pairs per lane
  const int lane = threadIdx.x & 63;
  const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (wid >= (int64_t)T * H) return;   // whole wave
  const int r = (int)(wid / H), h = (int)(wid - (int64_t)r * H);
  const bf16* xp = x + (int64_t)r * xs + (int64_t)h * HD;
  float v0[PPL], v1[PPL], ss = 0.f;
#pragma unroll
  for (int j = 0; j < PPL; ++j) {
    const int p = lane + 64 * j;
    v0[j] = v1[j] = 0.f;
    if (p < NP) {
      const bf16x2 t = *reinterpret_cast<const bf16x2*>(xp + 2 * p);
      v0[j] = (float)t[0];
      v1[j] = (float)t[1];
      ss += v0[j] * v0[j] + v1[j] * v1[j];
    }
  }
  if (w != nullptr) {
    const float inv = rsqrtf(wave_sum(ss) / HD + eps);
#pragma unroll
    for (int j = 0; j < PPL; ++j) {
      const int p = lane + 64 * j;
      if (p < NP) {
        v0[j] = (float)(bf16)((float)(bf16)(v0[j] * inv) * (float)w[2 * p]);
        v1[j] = (float)(bf16)((float)(bf16)(v1[j] * inv) * (float)w[2 * p + 1]);
      }
    }
  }
  bf16* op = out + (int64_t)(dst != nullptr ? dst[r] : r) * os + (int64_t)h * HD;
#pragma unroll
  for (int j = 0; j < PPL; ++j) {
    const int p = lane + 64 * j;
    if (p >= NP) continue;
    float a = v0[j], b = v1[j];
    if (cs != nullptr) {
      const float2 c = *reinterpret_cast<const float2*>(cs + ((int64_t)r * NP + p) * 2);
      a = v0[j] * c.x - v1[j] * c.y;
      b = v0[j] * c.y + v1[j] * c.x;
    }
    bf16x2 o;
    o[0] = (bf16)a;
    o[1] = (bf16)b;
    *reinterpret_cast<bf16x2*>(op + 2 * p) = o;
  }
}

OME_API int ome_qk_norm_rope(const void* x, int64_t xs, const void* w, const float* cs, int T, int H, int hd,
                             float eps, void* out, int64_t os, const int* dst, hipStream_t stream) {
  if (T <= 0 || H <= 0) return 0;
  if ((xs | os) & 1) return -3;
  const int64_t waves = (int64_t)T * H;
  dim3 grid((unsigned)((waves + 3) / 4));
  switch (hd) {
    case 64:
      qk_norm_rope_kernel<64><<<grid, 256, 0, stream>>>((const bf16*)x, xs, (const bf16*)w, cs, T, H, eps, (bf16*)out,
                                                        os, dst);
      break;
    case 128:
      qk_norm_rope_kernel<128><<<grid, 256, 0, stream>>>((const bf16*)x, xs, (const bf16*)w, cs, T, H, eps,
                                                         (bf16*)out, os, dst);
      break;
    case 256:
      qk_norm_rope_kernel<256><<<grid, 256, 0, stream>>>((const bf16*)x, xs, (const bf16*)w, cs, T, H, eps,
                                                         (bf16*)out, os, dst);
      break;
    default:
      return -2;
  }
  OME_CHECK_LAUNCH();
  return 0;
}


// ---- fp32 residual stream (decoders that keep x in fp32 for the whole stack) ----
// res[row] += s1 * x1[row] + s2 * x2[row] (either addend may be null: the outputs of the previous
// block's sublayer(s), bf16), stored back as fp32, then out[row] = bf16(res * rsqrt(mean(res^2)
// + eps) * w).  One 256-thread workgroup per row, any width: the sum is formed and written in
// pass one (with the square sum), pass two re-reads the row it just wrote (cache-hot).
// T: element type of the addends, the weight and the output (bf16, or float for fp32 models).
template <typename T>
__global__ __launch_bounds__(256) void residual_rmsnorm_kernel(float* __restrict__ res, int64_t res_stride,
                                                               const T* __restrict__ x1, int64_t x1_stride,
                                                               float s1, const T* __restrict__ x2,
                                                               int64_t x2_stride, float s2,
                                                               const T* __restrict__ w, T* __restrict__ out,
                                                               int64_t out_stride, int H, float eps) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  float* r = res + row * res_stride;
  const T* a = x1 != nullptr ? x1 + row * x1_stride : nullptr;
  const T* b = x2 != nullptr ? x2 + row * x2_stride : nullptr;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = r[i];
    if (a != nullptr) {
      float add = s1 * (float)a[i];
      if (b != nullptr) add += s2 * (float)b[i];
      v += add;
      r[i] = v;
    }
    ss += v * v;
  }
  const float tot = block_sum<256>(ss, red);
  const float rs = 1.f / sqrtf(tot / (float)H + eps);
  T* o = out + row * out_stride;
  for (int i = threadIdx.x; i < H; i += 256) o[i] = (T)(r[i] * rs * (float)w[i]);
}

OME_API int ome_residual_rmsnorm(float* res, int64_t res_stride, const void* x1, int64_t x1_stride, float s1,
                                 const void* x2, int64_t x2_stride, float s2, const void* w, void* out,
                                 int64_t out_stride, int rows, int H, float eps, int f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || (x1 == nullptr && x2 != nullptr)) return -2;
  if (f32)
    residual_rmsnorm_kernel<float><<<rows, 256, 0, stream>>>(res, res_stride, (const float*)x1, x1_stride, s1,
                                                             (const float*)x2, x2_stride, s2, (const float*)w,
                                                             (float*)out, out_stride, H, eps);
  else
    residual_rmsnorm_kernel<bf16><<<rows, 256, 0, stream>>>(res, res_stride, (const bf16*)x1, x1_stride, s1,
                                                            (const bf16*)x2, x2_stride, s2, (const bf16*)w,
                                                            (bf16*)out, out_stride, H, eps);
  OME_CHECK_LAUNCH();
  return 0;
}

// ------------------------------------------------------------------------------------------
// Post-norm step of an fp32 residual stream: res += norm(y) * w (+ b), the norm taken over the
// SUBLAYER OUTPUT y (not over the stream).  kind 0: layer norm ((y - mean) / sqrt(var + eps), var =
// mean squared deviation), kind 1: RMS norm (y / sqrt(mean(y^2) + eps)).  Statistics, scaling and
// the sum are fp32; `out` (optional) gets the updated stream rounded to T: the next GEMM's input.
// One workgroup per row; the row of y stays in registers (H <= 256 * PN_MAX) or is re-read.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void post_norm_add_kernel(float* __restrict__ res, int64_t res_stride,
                                                            const T* __restrict__ y, int64_t y_stride,
                                                            const T* __restrict__ w, const T* __restrict__ b,
                                                            T* __restrict__ out, int64_t out_stride, int H, float eps,
                                                            int kind) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* yr = y + row * y_stride;
  float* r = res + row * res_stride;
  float s = 0.f;
  if (kind == 0) {
    for (int i = threadIdx.x; i < H; i += 256) s += (float)yr[i];
    s = block_sum<256>(s, red);
  }
  const float mean = kind == 0 ? s / (float)H : 0.f;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float d = (float)yr[i] - mean;
    ss += d * d;
  }
  ss = block_sum<256>(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = ((float)yr[i] - mean) * rs * (float)w[i];
    if (b != nullptr) v += (float)b[i];
    v += r[i];
    r[i] = v;
    if (out != nullptr) out[row * out_stride + i] = (T)v;
  }
}

// bf16 rows of 8-element vectors held in registers (NCH vectors per thread): y is read once, with
// 16-byte loads; the fp32 stream is read and written as float4 pairs.
template <int NCH>
__global__ __launch_bounds__(256) void post_norm_add_vec_kernel(float* __restrict__ res, int64_t res_stride,
                                                                const bf16* __restrict__ y, int64_t y_stride,
                                                                const bf16* __restrict__ w, const bf16* __restrict__ b,
                                                                bf16* __restrict__ out, int64_t out_stride, int H,
                                                                float eps, int kind) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int nv = H >> 3;
  const bf16* yr = y + row * y_stride;
  float v[NCH][8];
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = threadIdx.x + k * 256;
    if (c < nv) {
      const bf16x8 t = *(const bf16x8*)(yr + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[k][j] = (float)t[j];
        s += v[k][j];
      }
    }
  }
  float mean = 0.f;
  if (kind == 0) mean = block_sum<256>(s, red) / (float)H;
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    if (threadIdx.x + k * 256 < nv) {
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        v[k][j] -= mean;
        ss += v[k][j] * v[k][j];
      }
    }
  }
  ss = block_sum<256>(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)H + eps);
  float* r = res + row * res_stride;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = threadIdx.x + k * 256;
    if (c < nv) {
      const bf16x8 wv = *(const bf16x8*)(w + c * 8);
      f32x4 r0 = *(const f32x4*)(r + c * 8), r1 = *(const f32x4*)(r + c * 8 + 4);
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = v[k][j] * rs * (float)wv[j];
      if (b != nullptr) {
        const bf16x8 bv = *(const bf16x8*)(b + c * 8);
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] += (float)bv[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        r0[j] += o[j];
        r1[j] += o[j + 4];
      }
      *(f32x4*)(r + c * 8) = r0;
      *(f32x4*)(r + c * 8 + 4) = r1;
      if (out != nullptr) {
        bf16x8 ov;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          ov[j] = (bf16)r0[j];
          ov[j + 4] = (bf16)r1[j];
        }
        *(bf16x8*)(out + row * out_stride + c * 8) = ov;
      }
    }
  }
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

OME_API int ome_post_norm_add(float* res, int64_t res_stride, const void* y, int64_t y_stride, const void* w,
                              const void* b, void* out, int64_t out_stride, int rows, int H, float eps, int kind,
                              int f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || kind < 0 || kind > 1) return -2;
  if (!f32 && H % 8 == 0 && H <= 8 * 256 * 8 && res_stride % 4 == 0 && y_stride % 8 == 0 && out_stride % 8 == 0 &&
      aligned16(res) && aligned16(y) && aligned16(w) && aligned16(b) && aligned16(out)) {
    const int nch = (H / 8 + 255) / 256;
#define PNA_VEC(N)                                                                                                 \
  post_norm_add_vec_kernel<N><<<rows, 256, 0, stream>>>(res, res_stride, (const bf16*)y, y_stride, (const bf16*)w, \
                                                        (const bf16*)b, (bf16*)out, out_stride, H, eps, kind)
    if (nch <= 1) PNA_VEC(1);
    else if (nch <= 2) PNA_VEC(2);
    else if (nch <= 4) PNA_VEC(4);
    else PNA_VEC(8);
#undef PNA_VEC
    OME_CHECK_LAUNCH();
    return 0;
  }
  if (f32)
    post_norm_add_kernel<float><<<rows, 256, 0, stream>>>(res, res_stride, (const float*)y, y_stride, (const float*)w,
                                                          (const float*)b, (float*)out, out_stride, H, eps, kind);
  else
    post_norm_add_kernel<bf16><<<rows, 256, 0, stream>>>(res, res_stride, (const bf16*)y, y_stride, (const bf16*)w,
                                                         (const bf16*)b, (bf16*)out, out_stride, H, eps, kind);
  OME_CHECK_LAUNCH();
  return 0;
}

// ------------------------------------------------------------------------------------------
// PolyNorm activation: out = a N(z) + b N(z^2) + c N(z^3) + e with element-wise powers and
// N(u) = u / sqrt(mean(u^2) + eps) over the row; coef = (a, b, c, e) fp32.  The three mean
// squares (of z, z^2, z^3) come from one pass in fp32, the second pass writes the sum.
// ------------------------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void polynorm_kernel(const T* __restrict__ z, int64_t z_stride,
                                                       const float* __restrict__ coef, T* __restrict__ out,
                                                       int64_t out_stride, int F, float eps) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const T* zr = z + row * z_stride;
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
  for (int i = threadIdx.x; i < F; i += 256) {
    const float v = (float)zr[i], v2 = v * v;
    s1 += v2;
    s2 += v2 * v2;
    s3 += v2 * v2 * v2;
  }
  s1 = block_sum<256>(s1, red);
  s2 = block_sum<256>(s2, red);
  s3 = block_sum<256>(s3, red);
  const float n = (float)F;
  const float r1 = coef[0] / sqrtf(s1 / n + eps), r2 = coef[1] / sqrtf(s2 / n + eps),
              r3 = coef[2] / sqrtf(s3 / n + eps), e = coef[3];
  for (int i = threadIdx.x; i < F; i += 256) {
    const float v = (float)zr[i];
    out[row * out_stride + i] = (T)(v * (r1 + v * (r2 + v * r3)) + e);
  }
}

template <int NCH>
__global__ __launch_bounds__(256) void polynorm_vec_kernel(const bf16* __restrict__ z, int64_t z_stride,
                                                           const float* __restrict__ coef, bf16* __restrict__ out,
                                                           int64_t out_stride, int F, float eps) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const int nv = F >> 3;
  const bf16* zr = z + row * z_stride;
  bf16x8 v[NCH];
  float s1 = 0.f, s2 = 0.f, s3 = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = threadIdx.x + k * 256;
    if (c < nv) {
      v[k] = *(const bf16x8*)(zr + c * 8);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = (float)v[k][j], x2 = x * x;
        s1 += x2;
        s2 += x2 * x2;
        s3 += x2 * x2 * x2;
      }
    }
  }
  s1 = block_sum<256>(s1, red);
  s2 = block_sum<256>(s2, red);
  s3 = block_sum<256>(s3, red);
  const float n = (float)F;
  const float r1 = coef[0] / sqrtf(s1 / n + eps), r2 = coef[1] / sqrtf(s2 / n + eps),
              r3 = coef[2] / sqrtf(s3 / n + eps), e = coef[3];
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = threadIdx.x + k * 256;
    if (c < nv) {
      bf16x8 o;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float x = (float)v[k][j];
        o[j] = (bf16)(x * (r1 + x * (r2 + x * r3)) + e);
      }
      *(bf16x8*)(out + row * out_stride + c * 8) = o;
    }
  }
}

OME_API int ome_polynorm(const void* z, int64_t z_stride, const float* coef, void* out, int64_t out_stride, int rows,
                         int F, float eps, int f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (F <= 0) return -2;
  if (!f32 && F % 8 == 0 && F <= 8 * 256 * 16 && z_stride % 8 == 0 && out_stride % 8 == 0 && aligned16(z) &&
      aligned16(out)) {
    const int nch = (F / 8 + 255) / 256;
#define PN_VEC(N) \
  polynorm_vec_kernel<N><<<rows, 256, 0, stream>>>((const bf16*)z, z_stride, coef, (bf16*)out, out_stride, F, eps)
    if (nch <= 1) PN_VEC(1);
    else if (nch <= 2) PN_VEC(2);
    else if (nch <= 4) PN_VEC(4);
    else if (nch <= 8) PN_VEC(8);
    else PN_VEC(16);
#undef PN_VEC
    OME_CHECK_LAUNCH();
    return 0;
  }
  if (f32)
    polynorm_kernel<float><<<rows, 256, 0, stream>>>((const float*)z, z_stride, coef, (float*)out, out_stride, F, eps);
  else
    polynorm_kernel<bf16><<<rows, 256, 0, stream>>>((const bf16*)z, z_stride, coef, (bf16*)out, out_stride, F, eps);
  OME_CHECK_LAUNCH();
  return 0;
}

// ------------------------------------------------------------------------------------------
// Row norm for any width and element type: out = norm(x) * w (+ b), kind 0 layer norm / 1 RMS
// norm, statistics in fp32.  TI: the input's type (an fp32 residual stream, or a projection's
// output), TO: the type of w, b and out.  One workgroup per row.
// ------------------------------------------------------------------------------------------
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void row_norm_kernel(const TI* __restrict__ x, int64_t x_stride,
                                                       const TO* __restrict__ w, const TO* __restrict__ b,
                                                       TO* __restrict__ out, int64_t out_stride, int H, float eps,
                                                       int kind) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const TI* xr = x + row * x_stride;
  float s = 0.f;
  if (kind == 0) {
    for (int i = threadIdx.x; i < H; i += 256) s += (float)xr[i];
    s = block_sum<256>(s, red);
  }
  const float mean = kind == 0 ? s / (float)H : 0.f;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float d = (float)xr[i] - mean;
    ss += d * d;
  }
  ss = block_sum<256>(ss, red);
  const float rs = 1.f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = ((float)xr[i] - mean) * rs * (float)w[i];
    if (b != nullptr) v += (float)b[i];
    out[row * out_stride + i] = (TO)v;
  }
}

OME_API int ome_row_norm(const void* x, int64_t x_stride, int x_f32, const void* w, const void* b, void* out,
                         int64_t out_stride, int rows, int H, float eps, int kind, int f32, hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || kind < 0 || kind > 1 || (f32 && !x_f32)) return -2;
  if (f32)
    row_norm_kernel<float, float><<<rows, 256, 0, stream>>>((const float*)x, x_stride, (const float*)w,
                                                            (const float*)b, (float*)out, out_stride, H, eps, kind);
  else if (x_f32)
    row_norm_kernel<float, bf16><<<rows, 256, 0, stream>>>((const float*)x, x_stride, (const bf16*)w, (const bf16*)b,
                                                           (bf16*)out, out_stride, H, eps, kind);
  else
    row_norm_kernel<bf16, bf16><<<rows, 256, 0, stream>>>((const bf16*)x, x_stride, (const bf16*)w, (const bf16*)b,
                                                          (bf16*)out, out_stride, H, eps, kind);
  OME_CHECK_LAUNCH();
  return 0;
}

// ------------------------------------------------------------------------------------------
// Pre-norm step of an fp32 residual stream with a token shift.  For row t of sequence s:
//   v[t]   = res_in[t] + s1 * x1[t] + s2 * x2[t] + bias       (either addend may be absent; bias:
//                                                            one row of width H for all rows, or null)
//   n[t]   = v[t] / sqrt(mean(v[t]^2) + eps) * (w_off + w)  (fp32; w_off = 1 for weights stored
//                                                            as the offset from one)
//   out[t] = n[t] + (n[t-1] - n[t]) * mu                     (rounded once, to T)
// n[t-1] of a sequence's first row of this step is the row kept per request slot in `state`
// [slots, H] fp32 (zeros when reset[s] is set); the step's last n of the sequence replaces it.
// The updated stream goes to a second buffer (res_out), so the workgroup of row t can form n[t-1]
// from the step's inputs without waiting for the workgroup of row t-1.  Only the workgroup of a
// sequence's first row touches the state: it reads the old row, then (after forming the n of the
// sequence's last row itself) writes the new one.  mu == nullptr: no shift (plain norm, no state).
// ------------------------------------------------------------------------------------------
namespace {
template <typename T>
__device__ __forceinline__ float shift_row_rs(const float* __restrict__ r, const T* __restrict__ a, float s1,
                                              const T* __restrict__ b, float s2, const T* __restrict__ c, int H,
                                              float eps, float* red) {
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = r[i];
    if (a != nullptr) v += s1 * (float)a[i];
    if (b != nullptr) v += s2 * (float)b[i];
    if (c != nullptr) v += (float)c[i];
    ss += v * v;
  }
  return 1.f / sqrtf(block_sum<256>(ss, red) / (float)H + eps);
}

template <typename T>
__device__ __forceinline__ float shift_val(const float* r, const T* a, float s1, const T* b, float s2, const T* c,
                                           int i) {
  float v = r[i];
  if (a != nullptr) v += s1 * (float)a[i];
  if (b != nullptr) v += s2 * (float)b[i];
  if (c != nullptr) v += (float)c[i];
  return v;
}

template <typename T>
__global__ __launch_bounds__(256) void shift_norm_kernel(
    const float* __restrict__ res_in, float* __restrict__ res_out, int64_t res_stride, const T* __restrict__ x1,
    int64_t x1_stride, float s1, const T* __restrict__ x2, int64_t x2_stride, float s2, const T* __restrict__ w,
    float w_off, const T* __restrict__ mu, float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slot, const int* __restrict__ reset, int S, T* __restrict__ out, int64_t out_stride,
    int H, float eps, const T* __restrict__ bias) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const float* r = res_in + row * res_stride;
  const T* a = x1 != nullptr ? x1 + row * x1_stride : nullptr;
  const T* b = x2 != nullptr ? x2 + row * x2_stride : nullptr;
  const float rs = shift_row_rs(r, a, s1, b, s2, bias, H, eps, red);
  float* ro = res_out + row * res_stride;
  T* o = out + row * out_stride;
  if (mu == nullptr) {
    for (int i = threadIdx.x; i < H; i += 256) {
      const float v = shift_val(r, a, s1, b, s2, bias, i);
      ro[i] = v;
      o[i] = (T)(v * rs * (w_off + (float)w[i]));
    }
    return;
  }
  int s = 0;
  while (s + 1 < S && cu[s + 1] <= (int)row) ++s;   // the sequence with cu[s] <= row < cu[s + 1]
  const int first = cu[s], last = cu[s + 1] - 1;
  if ((int)row != first) {   // the row before belongs to this step
    const float* rp = r - res_stride;
    const T* ap = a != nullptr ? a - x1_stride : nullptr;
    const T* bp = b != nullptr ? b - x2_stride : nullptr;
    const float rsp = shift_row_rs(rp, ap, s1, bp, s2, bias, H, eps, red);
    for (int i = threadIdx.x; i < H; i += 256) {
      const float v = shift_val(r, a, s1, b, s2, bias, i), wi = w_off + (float)w[i];
      const float n = v * rs * wi, np = shift_val(rp, ap, s1, bp, s2, bias, i) * rsp * wi;
      ro[i] = v;
      o[i] = (T)(n + (np - n) * (float)mu[i]);
    }
    return;
  }
  float* st = state + (int64_t)slot[s] * H;
  const bool fresh = reset[s] != 0;
  const int64_t d = last - first;   // rows from this one to the sequence's last of the step
  const float* rl = r + d * res_stride;
  const T* al = a != nullptr ? a + d * x1_stride : nullptr;
  const T* bl = b != nullptr ? b + d * x2_stride : nullptr;
  const float rsl = d > 0 ? shift_row_rs(rl, al, s1, bl, s2, bias, H, eps, red) : rs;
  for (int i = threadIdx.x; i < H; i += 256) {
    const float v = shift_val(r, a, s1, b, s2, bias, i), wi = w_off + (float)w[i];
    const float n = v * rs * wi, np = fresh ? 0.f : st[i];
    ro[i] = v;
    o[i] = (T)(n + (np - n) * (float)mu[i]);
    st[i] = d > 0 ? shift_val(rl, al, s1, bl, s2, bias, i) * rsl * wi : n;
  }
}
}  // namespace

// The same step for rows of 4-element vectors held in registers (H % 4 == 0, H <= 1024 * NCH,
// 16-byte aligned fp32 rows, 8-byte aligned bf16 rows): the stream, the addends and the row before
// are each read once, with vector loads.
namespace {
template <typename T>
__device__ __forceinline__ f32x4 sn_ld4(const T* p) {
  if constexpr (sizeof(T) == 4) {
    return *reinterpret_cast<const f32x4*>(p);
  } else {
    const bf16x4 t = *reinterpret_cast<const bf16x4*>(p);
    return f32x4{(float)t[0], (float)t[1], (float)t[2], (float)t[3]};
  }
}
template <typename T>
__device__ __forceinline__ void sn_st4(T* p, f32x4 v) {
  if constexpr (sizeof(T) == 4) {
    *reinterpret_cast<f32x4*>(p) = v;
  } else {
    *reinterpret_cast<bf16x4*>(p) = bf16x4{(bf16)v[0], (bf16)v[1], (bf16)v[2], (bf16)v[3]};
  }
}

// v = r + s1 a + s2 b + c of one row into registers; returns 1 / rms
template <typename T, int NCH>
__device__ __forceinline__ float sn_row(const float* __restrict__ r, const T* __restrict__ a, float s1,
                                        const T* __restrict__ b, float s2, const T* __restrict__ cb, int H, float eps,
                                        float* red, f32x4 (&v)[NCH]) {
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * 4;
    if (c < H) {
      f32x4 x = *reinterpret_cast<const f32x4*>(r + c);
      if (a != nullptr) x += s1 * sn_ld4<T>(a + c);
      if (b != nullptr) x += s2 * sn_ld4<T>(b + c);
      if (cb != nullptr) x += sn_ld4<T>(cb + c);
      v[k] = x;
      ss += x[0] * x[0] + x[1] * x[1] + x[2] * x[2] + x[3] * x[3];
    }
  }
  return 1.f / sqrtf(block_sum<256>(ss, red) / (float)H + eps);
}

template <typename T, int NCH>
__global__ __launch_bounds__(256) void shift_norm_vec_kernel(
    const float* __restrict__ res_in, float* __restrict__ res_out, int64_t res_stride, const T* __restrict__ x1,
    int64_t x1_stride, float s1, const T* __restrict__ x2, int64_t x2_stride, float s2, const T* __restrict__ w,
    float w_off, const T* __restrict__ mu, float* __restrict__ state, const int* __restrict__ cu,
    const int* __restrict__ slot, const int* __restrict__ reset, int S, T* __restrict__ out, int64_t out_stride,
    int H, float eps, const T* __restrict__ bias) {
  __shared__ float red[4];
  const int64_t row = blockIdx.x;
  const float* r = res_in + row * res_stride;
  const T* a = x1 != nullptr ? x1 + row * x1_stride : nullptr;
  const T* b = x2 != nullptr ? x2 + row * x2_stride : nullptr;
  f32x4 v[NCH], p[NCH];
  const float rs = sn_row<T, NCH>(r, a, s1, b, s2, bias, H, eps, red, v);
  float* ro = res_out + row * res_stride;
  T* o = out + row * out_stride;
  // kind of row: 0 no shift, 1 the row before is in this step, 2 first row of its sequence
  int kind = 0, s = 0, d = 0;
  float rsp = 0.f;
  if (mu != nullptr) {
    while (s + 1 < S && cu[s + 1] <= (int)row) ++s;
    kind = (int)row != cu[s] ? 1 : 2;
    d = cu[s + 1] - 1 - cu[s];
  }
  if (kind == 1) {
    rsp = sn_row<T, NCH>(r - res_stride, a != nullptr ? a - x1_stride : nullptr, s1,
                         b != nullptr ? b - x2_stride : nullptr, s2, bias, H, eps, red, p);
  } else if (kind == 2 && d > 0) {   // the sequence's last row of the step: the new state
    rsp = sn_row<T, NCH>(r + (int64_t)d * res_stride, a != nullptr ? a + (int64_t)d * x1_stride : nullptr, s1,
                         b != nullptr ? b + (int64_t)d * x2_stride : nullptr, s2, bias, H, eps, red, p);
  }
  float* st = kind == 2 ? state + (int64_t)slot[s] * H : nullptr;
  const bool fresh = kind == 2 && reset[s] != 0;
#pragma unroll
  for (int k = 0; k < NCH; ++k) {
    const int c = (threadIdx.x + 256 * k) * 4;
    if (c < H) {
      const f32x4 wi = sn_ld4<T>(w + c) + w_off;
      const f32x4 n = v[k] * rs * wi;
      *reinterpret_cast<f32x4*>(ro + c) = v[k];
      if (kind == 0) {
        sn_st4<T>(o + c, n);
      } else {
        const f32x4 m = sn_ld4<T>(mu + c);
        f32x4 np;
        if (kind == 1) np = p[k] * rsp * wi;
        else np = fresh ? f32x4{0.f, 0.f, 0.f, 0.f} : *reinterpret_cast<const f32x4*>(st + c);
        sn_st4<T>(o + c, n + (np - n) * m);
        if (kind == 2) *reinterpret_cast<f32x4*>(st + c) = d > 0 ? p[k] * rsp * wi : n;
      }
    }
  }
}
}  // namespace

OME_API int ome_shift_norm(const float* res_in, float* res_out, int64_t res_stride, const void* x1, int64_t x1_stride,
                           float s1, const void* x2, int64_t x2_stride, float s2, const void* w, float w_off,
                           const void* mu, float* state, const int* cu, const int* slot, const int* reset, int S,
                           void* out, int64_t out_stride, int rows, int H, float eps, int f32, const void* bias,
                           hipStream_t stream) {
  if (rows <= 0) return 0;
  if (H <= 0 || (mu != nullptr && (S <= 0 || state == nullptr))) return -2;
  const int esz = f32 ? 4 : 2;
  auto al = [](const void* p, int64_t stride, int e) { return (((uintptr_t)p | (uintptr_t)(stride * e)) & (4 * e - 1)) == 0; };
  if (H % 4 == 0 && H <= 8192 && al(res_in, res_stride, 4) && al(res_out, res_stride, 4) && al(x1, x1_stride, esz) &&
      al(x2, x2_stride, esz) && al(w, 0, esz) && al(mu, 0, esz) && al(out, out_stride, esz) && al(state, H, 4) &&
      al(bias, 0, esz)) {
#define SN_VEC(TT, N)                                                                                                \
  shift_norm_vec_kernel<TT, N><<<rows, 256, 0, stream>>>(res_in, res_out, res_stride, (const TT*)x1, x1_stride, s1,   \
                                                         (const TT*)x2, x2_stride, s2, (const TT*)w, w_off,           \
                                                         (const TT*)mu, state, cu, slot, reset, S, (TT*)out,          \
                                                         out_stride, H, eps, (const TT*)bias)
#define SN_PICK(TT)                 \
  do {                              \
    if (H <= 1024) SN_VEC(TT, 1);   \
    else if (H <= 2048) SN_VEC(TT, 2); \
    else if (H <= 4096) SN_VEC(TT, 4); \
    else SN_VEC(TT, 8);             \
  } while (0)
    if (f32) SN_PICK(float);
    else SN_PICK(bf16);
#undef SN_PICK
#undef SN_VEC
    OME_CHECK_LAUNCH();
    return 0;
  }
  if (f32)
    shift_norm_kernel<float><<<rows, 256, 0, stream>>>(res_in, res_out, res_stride, (const float*)x1, x1_stride, s1,
                                                       (const float*)x2, x2_stride, s2, (const float*)w, w_off,
                                                       (const float*)mu, state, cu, slot, reset, S, (float*)out,
                                                       out_stride, H, eps, (const float*)bias);
  else
    shift_norm_kernel<bf16><<<rows, 256, 0, stream>>>(res_in, res_out, res_stride, (const bf16*)x1, x1_stride, s1,
                                                      (const bf16*)x2, x2_stride, s2, (const bf16*)w, w_off,
                                                      (const bf16*)mu, state, cu, slot, reset, S, (bf16*)out,
                                                      out_stride, H, eps, (const bf16*)bias);
  OME_CHECK_LAUNCH();
  return 0;
}
