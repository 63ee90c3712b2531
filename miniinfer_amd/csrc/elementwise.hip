// Row-wise kernels of the decoder: embedding gather, (residual add +) RMS norm, SiLU*mul,
// and the fused per-head norm + rotary + cache write.  All arithmetic is 32-bit; values are
// rounded once, when they are stored in the activation dtype.
//
// Formulas restate tom-jerr/MiniInfer: layers/embedding.py:27 (gather), layers/layernorm.py:22-32
// and kernels/triton/rms_norm.py:84-101 (norm, add + norm), kernels/triton/silu_mul.py:33-37,
// models/fused_qwen3.py:98-105 with layers/position_encoding.py:91-117 (per-head norm, rotation),
// kvcache/memory_pool.py:55-56 (cache write).
#include "common.h"

// ---------------------------------------------------------------- embedding
// A negative id -(r + 1) stands for a token that an earlier kernel on the stream left in future[r] (the row of the
// last step's sampling output): the engine launches a step before it has read the tokens of the one before.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int H, int V, const int* __restrict__ future, int num_future) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 && future && -(id + 1) < num_future) id = future[-(id + 1)];
  const bool ok = id >= 0 && id < V;
  const T* row = table + (int64_t)(ok ? id : 0) * H;
  float* o = out + (int64_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = ok ? to_float(row[i]) : __builtin_nanf("");
}

MI_EXPORT int mi_embed(int dtype, const void* table, const int* ids, float* out, int T, int H, int V,
                       const int* future, int num_future, hipStream_t stream) {
  MI_REQUIRE(T >= 0 && H > 0 && V > 0 && num_future >= 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
  if (T == 0) return 0;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  if (dtype == MI_DTYPE_F32)
    embed_kernel<float><<<T, threads, 0, stream>>>((const float*)table, ids, out, H, V, future, num_future);
  else if (dtype == MI_DTYPE_BF16)
    embed_kernel<bf16><<<T, threads, 0, stream>>>((const bf16*)table, ids, out, H, V, future, num_future);
  else
    MI_FAIL("embed: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("embed");
  return 0;
}

// ---------------------------------------------------------------- (add +) RMS norm
// For output row i (source row s = rows ? rows[i] : i):
//   v = residual[s] + x[s]      (either may be absent)
//   residual[s] = v             (when write_back; never with `rows`)
//   y[i] = v * rsqrt(mean(v^2) + eps) * w
template <typename TX, typename TY>
__global__ void add_rmsnorm_kernel(const TX* __restrict__ x, float* __restrict__ residual,
                                   const float* __restrict__ w, TY* __restrict__ y, const int* __restrict__ rows,
                                   int N, float eps, int write_back) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int64_t s = rows ? rows[i] : i;
  const TX* xr = x ? x + s * N : nullptr;
  float* rr = residual ? residual + s * N : nullptr;
  TY* yr = y + (int64_t)i * N;

  float ss = 0.f;
  for (int c = threadIdx.x; c < N; c += blockDim.x) {
    float v = 0.f;
    if (rr) v = rr[c];
    if (xr) v += to_float(xr[c]);
    if (write_back) rr[c] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)N + eps);
  for (int c = threadIdx.x; c < N; c += blockDim.x) {
    float v;
    if (write_back) {
      v = rr[c];  // this thread wrote it above
    } else {
      v = 0.f;
      if (rr) v = rr[c];
      if (xr) v += to_float(xr[c]);
    }
    yr[c] = from_float<TY>(v * rstd * w[c]);
  }
}

// The same with every value held in registers: one read of x, residual and w (all loads issued together), one
// reduction, one write.  Each thread takes CH chunks of 4 consecutive elements; N must be a multiple of 4.
__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
__device__ __forceinline__ void load4(const bf16* p, float (&v)[4]) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
  v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void store4(bf16* p, const float (&v)[4]) {
  store2(p, v[0], v[1]);
  store2(p + 2, v[2], v[3]);
}

template <typename TX, typename TY, int CH>
__global__ void add_rmsnorm_reg_kernel(const TX* __restrict__ x, float* __restrict__ residual,
                                       const float* __restrict__ w, TY* __restrict__ y, const int* __restrict__ rows,
                                       int N, float eps, int write_back) {
  __shared__ float scratch[16];
  const int i = blockIdx.x;
  const int64_t s = rows ? rows[i] : i;
  const TX* xr = x ? x + s * N : nullptr;
  float* rr = residual ? residual + s * N : nullptr;
  TY* yr = y + (int64_t)i * N;
  float v[CH][4], wv[CH][4];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = 4 * (threadIdx.x + c * blockDim.x);
#pragma unroll
    for (int j = 0; j < 4; ++j) v[c][j] = 0.f, wv[c][j] = 0.f;
    if (e < N) {
      if (rr) load4(rr + e, v[c]);
      if (xr) {
        float t[4];
        load4(xr + e, t);
#pragma unroll
        for (int j = 0; j < 4; ++j) v[c][j] += t[j];
      }
      load4(w + e, wv[c]);
    }
  }
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = 4 * (threadIdx.x + c * blockDim.x);
    if (write_back && e < N) store4(rr + e, v[c]);
#pragma unroll
    for (int j = 0; j < 4; ++j) ss += v[c][j] * v[c][j];
  }
  ss = block_sum(ss, scratch);
  const float rstd = rsqrtf(ss / (float)N + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int e = 4 * (threadIdx.x + c * blockDim.x);
    if (e < N) {
      float o[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = v[c][j] * rstd * wv[c][j];
      store4(yr + e, o);
    }
  }
}

// x_dtype: dtype of x (ignored when x is null); y_dtype: dtype of y.
MI_EXPORT int mi_add_rmsnorm(int x_dtype, int y_dtype, const void* x, float* residual, const float* w, void* y,
                             const int* rows, int M, int N, float eps, int write_back, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && N > 0, "add_rmsnorm: bad sizes M=%d N=%d", M, N);
  MI_REQUIRE(x || residual, "add_rmsnorm: neither x nor residual given");
  MI_REQUIRE(!(write_back && rows), "add_rmsnorm: write_back with a row selection is not defined");
  MI_REQUIRE(!(write_back && !residual), "add_rmsnorm: write_back without a residual");
  if (M == 0) return 0;
  if (!x) x_dtype = MI_DTYPE_F32;
  // rows of up to 16384 elements, a multiple of 4: everything in registers; otherwise two passes over the row
  const int chunks = N / 4;
  const bool regs = (N % 4 == 0) && chunks <= 4 * 1024;
  const int ch = chunks <= 1024 ? (chunks <= 256 ? 1 : (chunks <= 512 ? 2 : 4)) : 4;
  const int rthreads = regs ? (((chunks + ch - 1) / ch + 63) / 64) * 64 : 0;
  const int threads = N >= 2048 ? 512 : (N >= 512 ? 256 : (N >= 128 ? 128 : 64));
#define LAUNCH(TX, TY)                                                                                         \
  do {                                                                                                         \
    if (regs && ch == 1)                                                                                       \
      add_rmsnorm_reg_kernel<TX, TY, 1><<<M, rthreads, 0, stream>>>((const TX*)x, residual, w, (TY*)y, rows, N, eps, write_back); \
    else if (regs && ch == 2)                                                                                  \
      add_rmsnorm_reg_kernel<TX, TY, 2><<<M, rthreads, 0, stream>>>((const TX*)x, residual, w, (TY*)y, rows, N, eps, write_back); \
    else if (regs)                                                                                             \
      add_rmsnorm_reg_kernel<TX, TY, 4><<<M, rthreads, 0, stream>>>((const TX*)x, residual, w, (TY*)y, rows, N, eps, write_back); \
    else                                                                                                       \
      add_rmsnorm_kernel<TX, TY><<<M, threads, 0, stream>>>((const TX*)x, residual, w, (TY*)y, rows, N, eps, write_back); \
  } while (0)
  if (x_dtype == MI_DTYPE_F32 && y_dtype == MI_DTYPE_F32) LAUNCH(float, float);
  else if (x_dtype == MI_DTYPE_BF16 && y_dtype == MI_DTYPE_BF16) LAUNCH(bf16, bf16);
  else if (x_dtype == MI_DTYPE_F32 && y_dtype == MI_DTYPE_BF16) LAUNCH(float, bf16);
  else if (x_dtype == MI_DTYPE_BF16 && y_dtype == MI_DTYPE_F32) LAUNCH(bf16, float);
  else MI_FAIL("add_rmsnorm: unknown dtypes %d %d", x_dtype, y_dtype);
#undef LAUNCH
  MI_CHECK_LAUNCH("add_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------- SiLU(gate) * up
// gu [M, 2I]: gate = first I columns, up = last I.  out [M, I].
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int M, int I) {
  const int64_t total = (int64_t)M * I;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = idx / I;
    const int c = (int)(idx - m * I);
    const float g = to_float(gu[m * 2 * I + c]);
    const float u = to_float(gu[m * 2 * I + I + c]);
    const float s = g / (1.f + expf(-g));
    out[idx] = from_float<T>(s * u);
  }
}

// the same, two pairs of columns per thread (I a multiple of 4: 64-bit and 128-bit accesses)
template <typename T>
__global__ void silu_mul4_kernel(const T* __restrict__ gu, T* __restrict__ out, int M, int I) {
  const int q = I / 4;
  const int64_t total = (int64_t)M * q;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = idx / q;
    const int c = 4 * (int)(idx - m * q);
    float g[4], u[4], r[4];
    load4(gu + m * 2 * I + c, g);
    load4(gu + m * 2 * I + I + c, u);
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = g[j] / (1.f + expf(-g[j])) * u[j];
    store4(out + m * I + c, r);
  }
}

MI_EXPORT int mi_silu_mul(int dtype, const void* gu, void* out, int M, int I, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && I > 0, "silu_mul: bad sizes M=%d I=%d", M, I);
  if (M == 0) return 0;
  if (I % 4 == 0) {
    const int64_t total4 = (int64_t)M * (I / 4);
    int64_t blocks4 = (total4 + 255) / 256;
    if (blocks4 > 65536) blocks4 = 65536;
    if (dtype == MI_DTYPE_F32)
      silu_mul4_kernel<float><<<(int)blocks4, 256, 0, stream>>>((const float*)gu, (float*)out, M, I);
    else if (dtype == MI_DTYPE_BF16)
      silu_mul4_kernel<bf16><<<(int)blocks4, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, M, I);
    else
      MI_FAIL("silu_mul: unknown dtype %d", dtype);
    MI_CHECK_LAUNCH("silu_mul");
    return 0;
  }
  const int64_t total = (int64_t)M * I;
  const int threads = 256;
  int64_t blocks = (total + threads - 1) / threads;
  if (blocks > 65536) blocks = 65536;
  if (dtype == MI_DTYPE_F32)
    silu_mul_kernel<float><<<(int)blocks, threads, 0, stream>>>((const float*)gu, (float*)out, M, I);
  else if (dtype == MI_DTYPE_BF16)
    silu_mul_kernel<bf16><<<(int)blocks, threads, 0, stream>>>((const bf16*)gu, (bf16*)out, M, I);
  else
    MI_FAIL("silu_mul: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("silu_mul");
  return 0;
}

// ---------------------------------------------------------------- per-head norm + rotary + cache write
// qkv [T, (nq + 2 nkv) d] with heads ordered q | k | v.  One wave per (token, head):
//   q heads: norm (if qw) and rotation (if cos_sin), written back in place;
//   k heads: the same with kw, written to the key pages (and back in place);
//   v heads: copied to the value pages.
// Key pages are [num_pages, nkv, P, d]; value pages are stored transposed, [num_pages, nkv, d, P], so that the
// attention kernels read runs of consecutive keys for one dim.  Token t goes to slot slots[t] = page * P + offset.
// cos_sin [max_pos, rotary_dim] = cos(pos * inv_freq_j) for j < rotary_dim/2, then sin(...).
// Pairs are (j, j + rotary_dim/2) within the first rotary_dim elements; the rest pass through.
template <typename T>
__global__ void qk_norm_rope_cache_kernel(T* __restrict__ qkv, int64_t row_stride, int nq, int nkv, int d,
                                          const float* __restrict__ qw, const float* __restrict__ kw, float eps,
                                          const float* __restrict__ cos_sin, int rotary_dim, int max_pos,
                                          const int* __restrict__ positions, T* __restrict__ k_pages,
                                          T* __restrict__ v_pages, const int* __restrict__ slots, int page_shift,
                                          int num_tokens) {
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int heads = nq + 2 * nkv;
  const int64_t wid = (int64_t)blockIdx.x * (blockDim.x / MI_WAVE) + threadIdx.x / MI_WAVE;
  if (wid >= (int64_t)num_tokens * heads) return;
  const int t = (int)(wid / heads);
  const int h = (int)(wid - (int64_t)t * heads);
  T* src = qkv + (int64_t)t * row_stride + (int64_t)h * d;
  const int P = 1 << page_shift;

  T* dst = nullptr;  // where the cache copy goes
  if (h >= nq && k_pages) {
    const int slot = slots[t];
    const int64_t page = slot >> page_shift;
    const int off = slot & (P - 1);
    const int g = (h - nq) % nkv;
    if (h < nq + nkv) {
      dst = k_pages + ((page * nkv + g) * P + off) * d;
    } else {  // value head: copy into the transposed page, element e of the head at [e][off]
      T* vdst = v_pages + (page * nkv + g) * (int64_t)d * P + off;
      for (int e = lane; e < d; e += MI_WAVE) vdst[(int64_t)e * P] = src[e];
    }
  }
  if (h >= nq + nkv) return;

  // every load that does not depend on another is issued first: the head's elements as rotation pairs
  // (j, j + half), two neighbouring pairs per lane, and the pass-through tail, the norm weights, the position
  const float* w = (h < nq) ? qw : kw;
  const int rd = cos_sin ? rotary_dim : 0;
  const int half = rd / 2;
  int pos = positions ? positions[t] : 0;
  pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
  const bool two = (half % 2 == 0);      // pairs j, j + 1 share 32-bit (bfloat16) or 64-bit accesses
  const int j = two ? 2 * lane : lane;   // first pair of this lane (half <= 128: one round)
  const int j2 = two ? j + 1 : j + 64;   // its second pair
  const bool ok1 = j < half, ok2 = j2 < half;
  float xa[2] = {0.f, 0.f}, xb[2] = {0.f, 0.f}, wa[2] = {1.f, 1.f}, wb[2] = {1.f, 1.f};
  if (two) {
    if (ok1) {
      load2(src + j, xa[0], xa[1]);
      load2(src + j + half, xb[0], xb[1]);
      if (w) {
        load2(w + j, wa[0], wa[1]);
        load2(w + j + half, wb[0], wb[1]);
      }
    }
  } else {
    if (ok1) { xa[0] = to_float(src[j]); xb[0] = to_float(src[j + half]); if (w) { wa[0] = w[j]; wb[0] = w[j + half]; } }
    if (ok2) { xa[1] = to_float(src[j2]); xb[1] = to_float(src[j2 + half]); if (w) { wa[1] = w[j2]; wb[1] = w[j2 + half]; } }
  }
  float xt[4], wt[4];                    // tail elements rd + lane + 64 c (d <= 256)
  float ss = xa[0] * xa[0] + xa[1] * xa[1] + xb[0] * xb[0] + xb[1] * xb[1];
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int e = rd + lane + 64 * c;
    const bool ok = e < d;
    xt[c] = ok ? to_float(src[e]) : 0.f;
    wt[c] = (ok && w) ? w[e] : 1.f;
    ss += xt[c] * xt[c];
  }
  float rstd = 1.f;
  if (w) rstd = rsqrtf(wave_sum(ss) / (float)d + eps);
  const float* cs = cos_sin ? cos_sin + (int64_t)pos * rotary_dim : nullptr;
  float cv[2] = {1.f, 1.f}, sv[2] = {0.f, 0.f};
  if (two) {
    if (ok1) {
      load2(cs + j, cv[0], cv[1]);
      load2(cs + half + j, sv[0], sv[1]);
    }
  } else {
    if (ok1) { cv[0] = cs[j]; sv[0] = cs[half + j]; }
    if (ok2) { cv[1] = cs[j2]; sv[1] = cs[half + j2]; }
  }
  float o1[2], o2[2];
#pragma unroll
  for (int c = 0; c < 2; ++c) {
    const float a = xa[c] * rstd * wa[c], b2 = xb[c] * rstd * wb[c];
    o1[c] = a * cv[c] - b2 * sv[c];
    o2[c] = b2 * cv[c] + a * sv[c];
  }
  if (two) {
    if (ok1) {
      store2(src + j, o1[0], o1[1]);
      store2(src + j + half, o2[0], o2[1]);
      if (dst) {
        store2(dst + j, o1[0], o1[1]);
        store2(dst + j + half, o2[0], o2[1]);
      }
    }
  } else {
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int jj = c == 0 ? j : j2;
      if (jj < half) {
        const T a = from_float<T>(o1[c]), b2 = from_float<T>(o2[c]);
        src[jj] = a;
        src[jj + half] = b2;
        if (dst) {
          dst[jj] = a;
          dst[jj + half] = b2;
        }
      }
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int e = rd + lane + 64 * c;
    if (e < d) {
      const T o = from_float<T>(xt[c] * rstd * wt[c]);
      src[e] = o;
      if (dst) dst[e] = o;
    }
  }
}

MI_EXPORT int mi_qk_norm_rope_cache(int dtype, void* qkv, int64_t row_stride, int num_tokens, int nq, int nkv, int d,
                                    const float* qw, const float* kw, float eps, const float* cos_sin,
                                    int rotary_dim, int max_pos, const int* positions, void* k_pages, void* v_pages,
                                    const int* slots, int page_size, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && nq > 0 && nkv >= 0 && d > 0, "qk_norm_rope_cache: bad sizes");
  MI_REQUIRE(d <= 256, "qk_norm_rope_cache: head size %d; this kernel takes at most 256", d);
  MI_REQUIRE(row_stride >= (int64_t)(nq + 2 * nkv) * d, "qk_norm_rope_cache: row stride %lld too small",
             (long long)row_stride);
  MI_REQUIRE(page_size > 0 && (page_size & (page_size - 1)) == 0, "qk_norm_rope_cache: page size %d is no power of two",
             page_size);
  if (cos_sin) {
    MI_REQUIRE(rotary_dim > 0 && rotary_dim % 2 == 0 && rotary_dim <= d, "qk_norm_rope_cache: rotary_dim %d for head %d",
               rotary_dim, d);
    MI_REQUIRE(positions != nullptr && max_pos > 0, "qk_norm_rope_cache: rotation without positions");
  }
  MI_REQUIRE((k_pages == nullptr) == (v_pages == nullptr), "qk_norm_rope_cache: key and value pages go together");
  MI_REQUIRE(!k_pages || slots, "qk_norm_rope_cache: cache write without slots");
  if (num_tokens == 0) return 0;
  int shift = 0;
  while ((1 << shift) < page_size) ++shift;
  const int waves_per_block = 4;
  const int64_t waves = (int64_t)num_tokens * (nq + 2 * nkv);
  const int blocks = (int)((waves + waves_per_block - 1) / waves_per_block);
  if (dtype == MI_DTYPE_F32)
    qk_norm_rope_cache_kernel<float><<<blocks, waves_per_block * MI_WAVE, 0, stream>>>(
        (float*)qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, rotary_dim, max_pos, positions, (float*)k_pages,
        (float*)v_pages, slots, shift, num_tokens);
  else if (dtype == MI_DTYPE_BF16)
    qk_norm_rope_cache_kernel<bf16><<<blocks, waves_per_block * MI_WAVE, 0, stream>>>(
        (bf16*)qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, rotary_dim, max_pos, positions, (bf16*)k_pages,
        (bf16*)v_pages, slots, shift, num_tokens);
  else
    MI_FAIL("qk_norm_rope_cache: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("qk_norm_rope_cache");
  return 0;
}
