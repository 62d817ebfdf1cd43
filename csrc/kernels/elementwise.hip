// Element-wise / gather kernels: SiLU-and-mul (K9), GELU-tanh-and-mul, vocab-parallel
// embedding gather (K13), residual add, and embedding pooling + L2 normalisation (K14).
// All memory-bound: 16-byte bf16x8 vectors per lane, grid-stride loops capped at
// 256 CUs x 8 blocks (Guideline 11).
#include "common.h"

__device__ __forceinline__ float silu(float x) { return x / (1.f + __expf(-x)); }
__device__ __forceinline__ float gelu_tanh(float x) {
  const float k0 = 0.7978845608028654f, k1 = 0.044715f;
  return 0.5f * x * (1.f + tanhf(k0 * (x + k1 * x * x * x)));
}

template <int ACT>
__global__ __launch_bounds__(256) void act_and_mul_kernel(const bf16* __restrict__ x, bf16* __restrict__ out,
                                                          int64_t rows, int I, bool il, float limit,
                                                          const float* __restrict__ rg = nullptr,
                                                          int64_t rg_stride = 0) {
  // rg (optional): one fp32 logit per row, the row's output is multiplied by its sigmoid
  // grid (column blocks, rows): no per-element 64-bit division, every lane one 16-B vector.
  // il: gate / up columns interleaved in 16-column blocks (the layout of a gate_up weight
  // interleaved for the fused SiLU*mul GEMM epilogue, ops.interleave_gate_up)
  const int nv = I >> 3;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t r = blockIdx.y;
  if (c >= nv) return;
  const bf16* xr = x + r * 2 * I;
  const int gcol = il ? ((c * 8) >> 4) * 32 + ((c * 8) & 15) : c * 8;
  const int ucol = il ? gcol + 16 : I + c * 8;
  bf16x8 g = ld8(xr + gcol), u = ld8(xr + ucol), o;
  const float rs = rg != nullptr ? 1.f / (1.f + expf(-rg[r * rg_stride])) : 1.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float gf = (float)g[j];
    if constexpr (ACT == 2 || ACT == 3) {
      // clamped SwiGLU / GeGELU: (clamp(u, -L, L) + 1) * g' * sigmoid(1.702 g'), g' = min(g, L);
      // L = 7 (GPT-OSS), 20 (Phi-3-small gegelu_limit)
      const float L = limit > 0.f ? limit : (ACT == 2 ? 7.f : 20.f);
      const float g2 = fminf(gf, L);
      const float u2 = fminf(fmaxf((float)u[j], -L), L);
      o[j] = (bf16)((u2 + 1.f) * g2 / (1.f + __expf(-1.702f * g2)) * rs);
    } else {
      const float a = ACT == 0 ? silu(gf) : gelu_tanh(gf);
      o[j] = (bf16)(a * (float)u[j] * rs);
    }
  }
  st8(out + r * I + c * 8, o);
}

// Non-gated activation (Starcoder2 / GPT-NeoX MLPs), in place on a contiguous bf16 tensor:
// ACT 1 = GELU-tanh, 3 = GELU (erf), 0 = SiLU, 4 = ReLU^2 (NemotronH, Persimmon, Arcee), 5 = ReLU (OPT)
template <int ACT>
__global__ __launch_bounds__(256) void act_kernel(bf16* __restrict__ x, int64_t nvec) {
  for (int64_t v = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; v < nvec; v += (int64_t)gridDim.x * blockDim.x) {
    bf16x8 a = ld8(x + v * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float f = (float)a[j];
      a[j] = (bf16)(ACT == 0   ? silu(f)
                     : ACT == 1 ? gelu_tanh(f)
                     : ACT == 4 ? fmaxf(f, 0.f) * fmaxf(f, 0.f)
                     : ACT == 5 ? fmaxf(f, 0.f)
                                : 0.5f * f * (1.f + erff(f * 0.7071067811865476f)));
    }
    st8(x + v * 8, a);
  }
}

static inline int grid_for(int64_t work, int nt) {
  int64_t g = (work + nt - 1) / nt;
  if (g > 2048) g = 2048;
  if (g < 1) g = 1;
  return (int)g;
}

// Any width (no vector loads): the gated activations for an intermediate size that is not a
// multiple of 8.  x [rows, 2I] = [gate | up].
template <typename T>
__global__ __launch_bounds__(256) void act_and_mul_any_kernel(const T* __restrict__ x, T* __restrict__ out,
                                                              int I, int act, float limit,
                                                              const float* __restrict__ rg = nullptr,
                                                              int64_t rg_stride = 0) {
  const int64_t r = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= I) return;
  const float gf = (float)x[r * 2 * I + c], uf = (float)x[r * 2 * I + I + c];
  float o;
  if (act == 2 || act == 3) {
    const float L = limit > 0.f ? limit : (act == 2 ? 7.f : 20.f);
    const float g2 = fminf(gf, L), u2 = fminf(fmaxf(uf, -L), L);
    o = (u2 + 1.f) * g2 / (1.f + expf(-1.702f * g2));
  } else {
    o = (act == 0 ? silu(gf) : gelu_tanh(gf)) * uf;
  }
  if (rg != nullptr) o *= 1.f / (1.f + expf(-rg[r * rg_stride]));
  out[r * I + c] = (T)o;
}

// act: 0 SiLU, 1 GELU-tanh, 2 clamped SwiGLU (GPT-OSS: limit 7), 3 Phi-3-small GeGELU (limit 20);
// limit > 0 replaces the clamp of act 2 / 3; | 16: interleaved gate/up (16-col blocks)
static int act_and_mul_launch(const void* x, void* out, int64_t rows, int I, int act, float limit, const float* rg,
                              int64_t rg_stride, hipStream_t stream) {
  if (rows <= 0) return 0;
  const bool il = (act & 16) != 0, f32 = (act & 32) != 0;   // | 32: fp32 elements
  act &= 15;
  if (il && I % 16) return -2;
  if (I % 8 || f32) {
    if (il) return -2;
    for (int64_t r0 = 0; r0 < rows; r0 += 65535) {
      const int64_t n = rows - r0 < 65535 ? rows - r0 : 65535;
      const dim3 g((I + 255) / 256, (unsigned)n);
      if (f32)
        act_and_mul_any_kernel<float><<<g, 256, 0, stream>>>((const float*)x + r0 * 2 * I, (float*)out + r0 * I, I,
                                                             act, limit, rg ? rg + r0 * rg_stride : nullptr,
                                                             rg_stride);
      else
        act_and_mul_any_kernel<bf16><<<g, 256, 0, stream>>>((const bf16*)x + r0 * 2 * I, (bf16*)out + r0 * I, I,
                                                            act, limit, rg ? rg + r0 * rg_stride : nullptr,
                                                            rg_stride);
    }
    OME_CHECK_LAUNCH();
    return 0;
  }
  for (int64_t r0 = 0; r0 < rows; r0 += 65535) {  // grid.y limit
    const int64_t n = rows - r0 < 65535 ? rows - r0 : 65535;
    const dim3 g((I / 8 + 255) / 256, (unsigned)n);
    const bf16* xp = (const bf16*)x + r0 * 2 * I;
    bf16* op = (bf16*)out + r0 * I;
    const float* rgp = rg ? rg + r0 * rg_stride : nullptr;
    if (act == 0)
      act_and_mul_kernel<0><<<g, 256, 0, stream>>>(xp, op, n, I, il, limit, rgp, rg_stride);
    else if (act == 1)
      act_and_mul_kernel<1><<<g, 256, 0, stream>>>(xp, op, n, I, il, limit, rgp, rg_stride);
    else if (act == 2)
      act_and_mul_kernel<2><<<g, 256, 0, stream>>>(xp, op, n, I, il, limit, rgp, rg_stride);
    else
      act_and_mul_kernel<3><<<g, 256, 0, stream>>>(xp, op, n, I, il, limit, rgp, rg_stride);
  }
  OME_CHECK_LAUNCH();
  return 0;
}

OME_API int ome_act_and_mul(const void* x, void* out, int64_t rows, int I, int act, float limit,
                            hipStream_t stream) {
  return act_and_mul_launch(x, out, rows, I, act, limit, nullptr, 0, stream);
}

// row_gate: fp32 logits, one per row (rows row_gate_stride apart): row r of the output is also
// multiplied by sigmoid(row_gate[r]) (a per-token gate on an always-on expert, applied ahead of
// its down projection, which is linear).
OME_API int ome_act_and_mul_rowgate(const void* x, void* out, int64_t rows, int I, int act, float limit,
                                    const float* row_gate, int64_t row_gate_stride, hipStream_t stream) {
  return act_and_mul_launch(x, out, rows, I, act, limit, row_gate, row_gate_stride, stream);
}

// Non-gated activation, any length and fp32 elements too (scalar accesses).
template <typename T>
__global__ __launch_bounds__(256) void act_any_kernel(T* __restrict__ x, int64_t n, int act) {
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (int64_t)gridDim.x * blockDim.x) {
    const float f = (float)x[i];
    x[i] = (T)(act == 0   ? f / (1.f + expf(-f))
               : act == 1 ? gelu_tanh(f)
               : act == 4 ? fmaxf(f, 0.f) * fmaxf(f, 0.f)
               : act == 5 ? fmaxf(f, 0.f)
                          : 0.5f * f * (1.f + erff(f * 0.7071067811865476f)));
  }
}

OME_API int ome_act_any(void* x, int64_t n, int act, int f32, hipStream_t stream) {
  if (n <= 0) return 0;
  if (act != 0 && act != 1 && act != 3 && act != 4 && act != 5) return -3;
  const int g = grid_for(n, 256);
  if (f32) act_any_kernel<float><<<g, 256, 0, stream>>>((float*)x, n, act);
  else act_any_kernel<bf16><<<g, 256, 0, stream>>>((bf16*)x, n, act);
  OME_CHECK_LAUNCH();
  return 0;
}

OME_API int ome_act(void* x, int64_t n, int act, hipStream_t stream) {
  if (n <= 0) return 0;
  if (n % 8) return -2;
  const int64_t nv = n / 8;
  const int g = grid_for(nv, 256);
  if (act == 0) act_kernel<0><<<g, 256, 0, stream>>>((bf16*)x, nv);
  else if (act == 1) act_kernel<1><<<g, 256, 0, stream>>>((bf16*)x, nv);
  else if (act == 4) act_kernel<4><<<g, 256, 0, stream>>>((bf16*)x, nv);
  else if (act == 5) act_kernel<5><<<g, 256, 0, stream>>>((bf16*)x, nv);
  else if (act == 3) act_kernel<3><<<g, 256, 0, stream>>>((bf16*)x, nv);
  else return -3;
  OME_CHECK_LAUNCH();
  return 0;
}

// out[t] = table[ids[t] - vocab_start] if the id falls in this rank's shard, else 0.
__global__ __launch_bounds__(256) void embedding_kernel(const int* __restrict__ ids, const bf16* __restrict__ table,
                                                        bf16* __restrict__ out, int T, int H, int vocab_start,
                                                        int vocab_end) {
  const int nv = H >> 3;
  for (int t = blockIdx.x; t < T; t += gridDim.x) {
    const int id = ids[t];
    const bool own = id >= vocab_start && id < vocab_end;
    const bf16* src = table + (int64_t)(own ? id - vocab_start : 0) * H;
    for (int c = threadIdx.x; c < nv; c += blockDim.x) {
      bf16x8 v = {};
      if (own) v = ld8(src + c * 8);
      st8(out + (int64_t)t * H + c * 8, v);
    }
  }
}

OME_API int ome_embedding(const int* ids, const void* table, void* out, int T, int H, int vocab_start,
                          int vocab_end, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H % 8) return -2;
  const int g = T < 4096 ? T : 4096;
  embedding_kernel<<<g, 256, 0, stream>>>(ids, (const bf16*)table, (bf16*)out, T, H, vocab_start, vocab_end);
  OME_CHECK_LAUNCH();
  return 0;
}

// Pooling for embedding models (--is-embedding): last-token or mean pooling over each sequence
// followed by optional L2 normalisation. hidden [T, H] bf16, cu_lens [S+1] -> out [S, H] f32.
__global__ __launch_bounds__(256) void pool_kernel(const bf16* __restrict__ hidden, const int* __restrict__ cu,
                                                   float* __restrict__ out, int H, int mode, int normalize) {
  __shared__ float red[4];
  const int s = blockIdx.x;
  const int b = cu[s], e = cu[s + 1];
  float ss = 0.f;
  for (int d = threadIdx.x; d < H; d += 256) {
    float v = 0.f;
    if (mode == 0) {
      v = (float)hidden[(int64_t)(e - 1) * H + d];
    } else if (mode == 2) {  // first token (CLS pooling: BERT / XLM-RoBERTa encoders)
      v = (float)hidden[(int64_t)b * H + d];
    } else {
      for (int t = b; t < e; ++t) v += (float)hidden[(int64_t)t * H + d];
      v /= (float)(e - b > 0 ? e - b : 1);
    }
    out[(int64_t)s * H + d] = v;
    ss += v * v;
  }
  if (!normalize) return;
  ss = block_sum<256>(ss, red);
  const float inv = 1.f / fmaxf(sqrtf(ss), 1e-12f);
  for (int d = threadIdx.x; d < H; d += 256) out[(int64_t)s * H + d] *= inv;
}

OME_API int ome_pool(const void* hidden, const int* cu_lens, void* out, int S, int H, int mode, int normalize,
                     hipStream_t stream) {
  if (S <= 0) return 0;
  pool_kernel<<<S, 256, 0, stream>>>((const bf16*)hidden, cu_lens, (float*)out, H, mode, normalize);
  OME_CHECK_LAUNCH();
  return 0;
}

// Overlapped scheduling: the next step is enqueued before the previous step's sampled ids
// reach the host, so rows whose input token is still "pending" take it from the previous
// step's device output: ids[i] = prev[src[i]] when src[i] >= 0 (one tiny kernel, no sync).
__global__ void fill_pending_kernel(int* __restrict__ ids, const int* __restrict__ src, const int* __restrict__ prev,
                                    int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    const int s = src[i];
    if (s >= 0) ids[i] = prev[s];
  }
}

OME_API int ome_fill_pending(int* ids, const int* src, const int* prev, int n, hipStream_t stream) {
  if (n <= 0) return 0;
  fill_pending_kernel<<<(n + 255) / 256, 256, 0, stream>>>(ids, src, prev, n);
  OME_CHECK_LAUNCH();
  return 0;
}

// Byte copy between any two device-visible addresses, one of which may be pinned host memory
// mapped into the GPU's address space (hipHostMalloc).  The per-step metadata H2D and the sampled
// ids D2H go through this kernel instead of hipMemcpyAsync, so every per-step transfer is a plain
// kernel dispatch on the compute stream (no copy-engine / runtime blit path, no per-step pinning).
__global__ __launch_bounds__(256) void copy_mapped_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                          int64_t n16, const unsigned char* __restrict__ src_tail,
                                                          unsigned char* __restrict__ dst_tail, int tail) {
  const int64_t i0 = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (int64_t i = i0; i < n16; i += (int64_t)gridDim.x * blockDim.x) dst[i] = src[i];
  if (i0 < tail) dst_tail[i0] = src_tail[i0];
}

OME_API int ome_copy_mapped(const void* src, void* dst, int64_t nbytes, hipStream_t stream) {
  if (nbytes <= 0) return 0;
  // 16-B vectors when both ends are 16-B aligned, bytes otherwise
  const bool vec = ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0);
  const int64_t n16 = vec ? nbytes / 16 : 0;
  const int64_t tail = nbytes - n16 * 16;
  if (tail > (1 << 20)) return -2;  // unaligned bulk copies are not this kernel's job
  const int64_t work = n16 > tail ? n16 : tail;
  int grid = (int)((work + 255) / 256);
  grid = grid < 1 ? 1 : (grid > 1024 ? 1024 : grid);
  if (tail > (int64_t)grid * 256) grid = (int)((tail + 255) / 256);
  copy_mapped_kernel<<<grid, 256, 0, stream>>>((const uint4*)src, (uint4*)dst, n16,
                                               (const unsigned char*)src + n16 * 16, (unsigned char*)dst + n16 * 16,
                                               (int)tail);
  OME_CHECK_LAUNCH();
  return 0;
}

// Device address of a pinned host allocation (identity on ROCm for hipHostMalloc memory).
OME_API int ome_host_device_ptr(void* host, void** dev) {
  return hipHostGetDevicePointer(dev, host, 0) == hipSuccess ? 0 : -1;
}


// fp32 rows table[ids] * scale: the start of an fp32 residual stream (ids outside [0, V): zeros)
template <typename T>
__global__ __launch_bounds__(256) void embedding_f32_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                                            float* __restrict__ out, int H, int V, float scale) {
  const int64_t t = blockIdx.x;
  const int id = ids[t];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (int64_t)(ok ? id : 0) * H;
  for (int i = threadIdx.x; i < H; i += 256) out[t * H + i] = ok ? (float)row[i] * scale : 0.f;
}

OME_API int ome_embedding_f32(const int* ids, const void* table, float* out, int T, int H, int V, float scale,
                              int f32, hipStream_t stream) {
  if (T <= 0) return 0;
  if (f32) embedding_f32_kernel<float><<<T, 256, 0, stream>>>(ids, (const float*)table, out, H, V, scale);
  else embedding_f32_kernel<bf16><<<T, 256, 0, stream>>>(ids, (const bf16*)table, out, H, V, scale);
  OME_CHECK_LAUNCH();
  return 0;
}

// fp32 rows table[id] * scale + pair[r] with a hashed token-pair row r = (previous id * mul_prev +
// id * mul_cur) mod buckets; a sequence's first token takes row `buckets` (the table's last).  The
// id before a chunk's first row is state[slot] (one int per request slot); the workgroup of that row
// reads it, then stores the chunk's last id there (no other workgroup touches the slot's entry).
// Rows of sequence s are cu[s] .. cu[s+1]-1; reset[s] != 0: the sequence starts in this step.
template <typename T>
__global__ __launch_bounds__(256) void pair_embedding_f32_kernel(
    const int* __restrict__ ids, const T* __restrict__ table, const T* __restrict__ pair, float* __restrict__ out,
    int* __restrict__ state, int H, int V, float scale, int buckets, long long mul_prev, long long mul_cur,
    const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ reset, int S) {
  const int64_t t = blockIdx.x;
  int s = 0;
  while (s + 1 < S && cu[s + 1] <= (int)t) ++s;   // the sequence with cu[s] <= t < cu[s + 1]
  const bool head = (int)t == cu[s];
  const int id = ids[t];
  const bool first = head && reset[s] != 0;
  const int prev = head ? (first ? 0 : state[slot[s]]) : ids[t - 1];
  long long r = ((long long)prev * mul_prev + (long long)id * mul_cur) % (long long)buckets;
  if (r < 0) r += buckets;
  if (first) r = buckets;
  const bool ok = id >= 0 && id < V;
  const T* row = table + (int64_t)(ok ? id : 0) * H;
  const T* prow = pair + r * H;
  for (int i = threadIdx.x; i < H; i += 256) out[t * H + i] = ok ? (float)row[i] * scale + (float)prow[i] : 0.f;
  if (head) {
    __syncthreads();   // every thread has read the old entry
    if (threadIdx.x == 0) state[slot[s]] = ids[cu[s + 1] - 1];
  }
}

OME_API int ome_pair_embedding_f32(const int* ids, const void* table, const void* pair, float* out, int* state, int T,
                                   int H, int V, float scale, int buckets, int64_t mul_prev, int64_t mul_cur,
                                   const int* cu, const int* slot, const int* reset, int S, int f32,
                                   hipStream_t stream) {
  if (T <= 0) return 0;
  if (buckets <= 0 || S <= 0) return -2;
  if (f32)
    pair_embedding_f32_kernel<float><<<T, 256, 0, stream>>>(ids, (const float*)table, (const float*)pair, out, state, H,
                                                            V, scale, buckets, mul_prev, mul_cur, cu, slot, reset, S);
  else
    pair_embedding_f32_kernel<bf16><<<T, 256, 0, stream>>>(ids, (const bf16*)table, (const bf16*)pair, out, state, H,
                                                           V, scale, buckets, mul_prev, mul_cur, cu, slot, reset, S);
  OME_CHECK_LAUNCH();
  return 0;
}

// Combine of a two-map (differential) attention.  a [T, 2 H, D]: per kv group g of R query heads,
// first the R outputs of map 1, then the R outputs of map 2 (head h = g R + r: a1 = a[(2 g) R + r],
// a2 = a[(2 g + 1) R + r]).  out[t, h, :] = o / sqrt(mean(o^2) + eps) * out_scale with o = a1 - lam a2
// over the first vdim <= D columns (fp32, one rounding); out is contiguous [T, H * vdim].  One wave
// per (row, head), vdim <= 64 * DN_MAX.
constexpr int DN_MAX = 4;
template <typename T>
__global__ __launch_bounds__(256) void diff_head_norm_kernel(const T* __restrict__ a, T* __restrict__ out, int H, int R,
                                                             int D, int vdim, float lam, float eps, float out_scale) {
  const int64_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  for (int h = blockIdx.y * 4 + wave; h < H; h += 4 * gridDim.y) {
    const int g = h / R, r = h - g * R;
    const T* a1 = a + (t * 2 * H + (int64_t)(2 * g) * R + r) * D;
    const T* a2 = a1 + (int64_t)R * D;
    float o[DN_MAX];
    float ss = 0.f;
#pragma unroll
    for (int k = 0; k < DN_MAX; ++k) {
      const int d = lane + 64 * k;
      o[k] = d < vdim ? (float)a1[d] - lam * (float)a2[d] : 0.f;
      ss += o[k] * o[k];
    }
    const float rs = out_scale / sqrtf(wave_sum(ss) / (float)vdim + eps);
    T* op = out + (t * H + h) * vdim;
#pragma unroll
    for (int k = 0; k < DN_MAX; ++k) {
      const int d = lane + 64 * k;
      if (d < vdim) op[d] = (T)(o[k] * rs);
    }
  }
}

OME_API int ome_diff_head_norm(const void* a, void* out, int T, int H, int R, int D, int vdim, float lam, float eps,
                               float out_scale, int f32, hipStream_t stream) {
  if (T <= 0) return 0;
  if (H <= 0 || R <= 0 || H % R || vdim <= 0 || vdim > D || vdim > 64 * DN_MAX) return -2;
  const dim3 grid(T, T >= 1024 ? 1 : (H + 3) / 4);
  if (f32)
    diff_head_norm_kernel<float><<<grid, 256, 0, stream>>>((const float*)a, (float*)out, H, R, D, vdim, lam, eps,
                                                           out_scale);
  else
    diff_head_norm_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)a, (bf16*)out, H, R, D, vdim, lam, eps,
                                                          out_scale);
  OME_CHECK_LAUNCH();
  return 0;
}

// Output gate of an attention layer: out[t, h * vdim + d] = o[t, h, d] * gate(g[t, h * vdim + d]),
// d < vdim <= D (o's head rows are D wide; the padding beyond vdim is dropped).  kind 0: sigmoid,
// 1: SiLU.
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(const T* __restrict__ o, const T* __restrict__ g,
                                                        int64_t g_stride, T* __restrict__ out, int H, int D,
                                                        int vdim, int kind) {
  const int64_t t = blockIdx.x;
  const int n = H * vdim;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int h = i / vdim, d = i - h * vdim;
    const float gv = (float)g[t * g_stride + i];
    const float sg = 1.f / (1.f + expf(-gv));
    out[t * n + i] = (T)((float)o[(t * H + h) * D + d] * (kind == 0 ? sg : gv * sg));
  }
}

OME_API int ome_head_gate(const void* o, const void* g, int64_t g_stride, void* out, int T, int H, int D, int vdim,
                          int kind, int f32, hipStream_t stream) {
  if (T <= 0) return 0;
  if (vdim <= 0 || vdim > D) return -2;
  if (f32)
    head_gate_kernel<float><<<T, 256, 0, stream>>>((const float*)o, (const float*)g, g_stride, (float*)out, H, D, vdim,
                                                   kind);
  else
    head_gate_kernel<bf16><<<T, 256, 0, stream>>>((const bf16*)o, (const bf16*)g, g_stride, (bf16*)out, H, D, vdim,
                                                  kind);
  OME_CHECK_LAUNCH();
  return 0;
}

// Per-token gated side input: out[t, j] = gelu_tanh(g[t, j]) * table[ids[t], col0 + j], j < n
// (g: a projection's output; table: a second embedding table whose row holds every layer's part,
// this layer's starting at column col0).  Product in fp32, one rounding.
template <typename T>
__global__ __launch_bounds__(256) void gelu_gather_mul_kernel(const T* __restrict__ g, int64_t g_stride,
                                                              const int* __restrict__ ids,
                                                              const T* __restrict__ table, int64_t t_stride, int V,
                                                              int col0, T* __restrict__ out, int n, int64_t total) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= total) return;
  const int64_t t = i / n;
  const int j = (int)(i - t * n);
  int id = ids[t];
  id = id < 0 ? 0 : (id >= V ? V - 1 : id);
  out[i] = (T)(gelu_tanh((float)g[t * g_stride + j]) * (float)table[(int64_t)id * t_stride + col0 + j]);
}

OME_API int ome_gelu_gather_mul(const void* g, int64_t g_stride, const int* ids, const void* table, int64_t t_stride,
                                int V, int col0, void* out, int T, int n, int f32, hipStream_t stream) {
  if (T <= 0 || n <= 0) return 0;
  const int64_t total = (int64_t)T * n;
  const int blocks = (int)((total + 255) / 256);
  if (f32)
    gelu_gather_mul_kernel<float><<<blocks, 256, 0, stream>>>((const float*)g, g_stride, ids, (const float*)table,
                                                              t_stride, V, col0, (float*)out, n, total);
  else
    gelu_gather_mul_kernel<bf16><<<blocks, 256, 0, stream>>>((const bf16*)g, g_stride, ids, (const bf16*)table,
                                                             t_stride, V, col0, (bf16*)out, n, total);
  OME_CHECK_LAUNCH();
  return 0;
}

// Rows of a mixture of experts whose router weight scales the expert's INPUT: out[t * k + j, :] =
// w[t, j] * x[t, :] (fp32 product, one rounding) -- the expanded, pre-scaled rows the grouped GEMM
// then sorts by expert.
template <typename T>
__global__ __launch_bounds__(256) void scale_rows_kernel(const T* __restrict__ x, int64_t x_stride,
                                                         const float* __restrict__ w, int k, T* __restrict__ out,
                                                         int H) {
  const int64_t r = blockIdx.x;            // expanded row t * k + j
  const float wv = w[r];
  const T* xr = x + (r / k) * x_stride;
  for (int i = threadIdx.x; i < H; i += 256) out[r * H + i] = (T)(wv * (float)xr[i]);
}

OME_API int ome_scale_rows(const void* x, int64_t x_stride, const float* w, int k, void* out, int T, int H, int f32,
                           hipStream_t stream) {
  if (T <= 0 || k <= 0) return 0;
  if (f32)
    scale_rows_kernel<float><<<T * k, 256, 0, stream>>>((const float*)x, x_stride, w, k, (float*)out, H);
  else
    scale_rows_kernel<bf16><<<T * k, 256, 0, stream>>>((const bf16*)x, x_stride, w, k, (bf16*)out, H);
  OME_CHECK_LAUNCH();
  return 0;
}
