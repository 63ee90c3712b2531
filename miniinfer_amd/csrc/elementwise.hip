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
// Optional parts of the gather, for model frames that ask for them: `scale` multiplies the row, and a second
// table `pos_table` [max_pos, H] adds the row of the token's position (learned absolute positions).
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, float* __restrict__ out,
                             int H, int V, const int* __restrict__ future, int num_future, float scale,
                             const T* __restrict__ pos_table, const int* __restrict__ positions, int max_pos) {
  const int t = blockIdx.x;
  int id = ids[t];
  if (id < 0 && future && -(id + 1) < num_future) id = future[-(id + 1)];
  bool ok = id >= 0 && id < V;
  const T* row = table + (int64_t)(ok ? id : 0) * H;
  const T* prow = nullptr;
  if (pos_table) {
    const int p = positions[t];
    ok = ok && p >= 0 && p < max_pos;
    prow = pos_table + (int64_t)(ok ? p : 0) * H;
  }
  float* o = out + (int64_t)t * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_float(row[i]) * scale;
    if (prow) v += to_float(prow[i]);
    o[i] = ok ? v : __builtin_nanf("");
  }
}

MI_EXPORT int mi_embed(int dtype, const void* table, const int* ids, float* out, int T, int H, int V,
                       const int* future, int num_future, float scale, const void* pos_table, const int* positions,
                       int max_pos, hipStream_t stream) {
  MI_REQUIRE(T >= 0 && H > 0 && V > 0 && num_future >= 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
  MI_REQUIRE(!pos_table || (positions && max_pos > 0), "embed: a position table needs positions");
  if (T == 0) return 0;
  const int threads = H >= 1024 ? 256 : (H >= 256 ? 128 : 64);
  if (dtype == MI_DTYPE_F32)
    embed_kernel<float><<<T, threads, 0, stream>>>((const float*)table, ids, out, H, V, future, num_future, scale,
                                                   (const float*)pos_table, positions, max_pos);
  else if (dtype == MI_DTYPE_BF16)
    embed_kernel<bf16><<<T, threads, 0, stream>>>((const bf16*)table, ids, out, H, V, future, num_future, scale,
                                                  (const bf16*)pos_table, positions, max_pos);
  else
    MI_FAIL("embed: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("embed");
  return 0;
}

// ---------------------------------------------------------------- logits: scale and soft cap, in place
// x = x * scale; with cap > 0 then x = cap * tanh(x / cap).  32-bit logits [R, V] with row stride ld.
__global__ void logit_transform_kernel(float* __restrict__ x, int64_t ld, int V, float scale, float cap) {
  float* row = x + (int64_t)blockIdx.y * ld;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < V; i += gridDim.x * blockDim.x) {
    float v = row[i] * scale;
    if (cap > 0.f) v = cap * tanhf(v / cap);
    row[i] = v;
  }
}

MI_EXPORT int mi_logit_transform(float* x, int64_t ld, int R, int V, float scale, float cap, hipStream_t stream) {
  MI_REQUIRE(R >= 0 && V > 0 && ld >= V && cap >= 0.f, "logit_transform: bad sizes R=%d V=%d", R, V);
  MI_REQUIRE(R <= 65535, "logit_transform: %d rows; the grid takes at most 65535", R);
  if (R == 0) return 0;
  const int bx = (V + 1023) / 1024 < 64 ? (V + 1023) / 1024 : 64;
  logit_transform_kernel<<<dim3(bx, R), 256, 0, stream>>>(x, ld, V, scale, cap);
  MI_CHECK_LAUNCH("logit_transform");
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

// ---------------------------------------------------------------- bias of a projection
// y[m][n] += b[n], in 32-bit, for projections that carry a bias (the products themselves have none).
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, int64_t ld, const T* __restrict__ b, int M, int N) {
  const int64_t total = (int64_t)M * N;
  for (int64_t idx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (int64_t)gridDim.x * blockDim.x) {
    const int64_t m = idx / N;
    const int n = (int)(idx - m * N);
    y[m * ld + n] = from_float<T>(to_float(y[m * ld + n]) + to_float(b[n]));
  }
}

MI_EXPORT int mi_add_bias(int dtype, void* y, int64_t ld, const void* b, int M, int N, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && N > 0 && ld >= N, "add_bias: bad sizes M=%d N=%d ld=%lld", M, N, (long long)ld);
  if (M == 0) return 0;
  int64_t blocks = ((int64_t)M * N + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (dtype == MI_DTYPE_F32)
    add_bias_kernel<float><<<(int)blocks, 256, 0, stream>>>((float*)y, ld, (const float*)b, M, N);
  else if (dtype == MI_DTYPE_BF16)
    add_bias_kernel<bf16><<<(int)blocks, 256, 0, stream>>>((bf16*)y, ld, (const bf16*)b, M, N);
  else
    MI_FAIL("add_bias: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("add_bias");
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

// The same for a product whose operand was an RMS norm's first half (bfloat16(residual * weight), with the sums of
// squares of each row left in parts: see gemm_skinny.hip, NormHalves): the norm's missing factor,
// rsqrt(sum_p row_ss[p][m] / K + eps), scales row m of gate and up before the activation.  Grid (column blocks, M).
template <typename T>
__global__ void silu_mul_scaled_kernel(const T* __restrict__ gu, T* __restrict__ out, int I,
                                       const float* __restrict__ row_ss, int ss_parts, int ss_row, float eps, int K) {
  __shared__ float scratch[16];
  const int m = blockIdx.y;
  float part = 0.f;
  for (int p = threadIdx.x; p < ss_parts; p += blockDim.x) part += row_ss[(int64_t)p * ss_row + m];
  const float rstd = rsqrtf(block_sum(part, scratch) / (float)K + eps);
  const int q = I / 4;
  for (int c4 = blockIdx.x * blockDim.x + threadIdx.x; c4 < q; c4 += gridDim.x * blockDim.x) {
    const int c = 4 * c4;
    float g[4], u[4], r[4];
    load4(gu + (int64_t)m * 2 * I + c, g);
    load4(gu + (int64_t)m * 2 * I + I + c, u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const float gs = g[j] * rstd;
      r[j] = gs / (1.f + expf(-gs)) * (u[j] * rstd);
    }
    store4(out + (int64_t)m * I + c, r);
  }
}

MI_EXPORT int mi_silu_mul_scaled(int dtype, const void* gu, void* out, int M, int I, const float* row_ss, int ss_parts,
                                 int ss_row, float eps, int K, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && M <= 65535 && I > 0 && I % 4 == 0, "silu_mul_scaled: M=%d I=%d (I must be a multiple of 4)", M, I);
  MI_REQUIRE(row_ss && ss_parts > 0 && ss_row >= M && K > 0, "silu_mul_scaled: parts=%d rows per part=%d K=%d", ss_parts,
             ss_row, K);
  if (M == 0) return 0;
  const dim3 grid((I / 4 + 255) / 256, M);
  if (dtype == MI_DTYPE_F32)
    silu_mul_scaled_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, I, row_ss, ss_parts, ss_row,
                                                            eps, K);
  else if (dtype == MI_DTYPE_BF16)
    silu_mul_scaled_kernel<bf16><<<grid, 256, 0, stream>>>((const bf16*)gu, (bf16*)out, I, row_ss, ss_parts, ss_row, eps,
                                                           K);
  else
    MI_FAIL("silu_mul_scaled: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("silu_mul_scaled");
  return 0;
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
                                          int num_tokens, int heads) {
  // heads = nq + 2 nkv, or nq + nkv when value_cache_write_kernel copies the values
  const int lane = threadIdx.x & (MI_WAVE - 1);
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

// The same norm and rotation for many tokens whose heads are rotated whole (rotary_dim == d, or no rotation) and
// whose values go through value_cache_write_kernel.  LPH lanes share a head: a lane takes 4 neighbouring rotation
// pairs (j .. j + 3, each with its partner d/2 further on) in 64-bit or 128-bit accesses, so a wave holds 64 / LPH
// heads of one token at a time, and two such sets in flight.  LPH is the power of two >= d / 8.
template <typename T, int LPH>
__device__ __forceinline__ void qk_norm_rope_many_body(int block, T* __restrict__ qkv, int64_t row_stride, int nq,
                                                       int nkv, int d, const float* __restrict__ qw,
                                                       const float* __restrict__ kw, float eps,
                                                       const float* __restrict__ cos_sin, int max_pos,
                                                       const int* __restrict__ positions, T* __restrict__ k_pages,
                                                       const int* __restrict__ slots, int page_shift, int num_tokens) {
  constexpr int HPS = MI_WAVE / LPH;     // heads per set
  constexpr int SETS = 2;
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int sub = lane / LPH, ln = lane % LPH;
  const int heads = nq + nkv;
  const int groups = (heads + HPS * SETS - 1) / (HPS * SETS);
  const int64_t wid = (int64_t)block * (blockDim.x / MI_WAVE) + threadIdx.x / MI_WAVE;
  if (wid >= (int64_t)num_tokens * groups) return;
  const int t = (int)(wid / groups);
  const int h0 = (int)(wid - (int64_t)t * groups) * HPS * SETS;
  const int half = d / 2;
  const int j = 4 * ln;
  const bool ok = j < half;
  int pos = (cos_sin && positions) ? positions[t] : 0;
  const int slot = k_pages ? slots[t] : 0;
  T* row = qkv + (int64_t)t * row_stride;
  float xa[SETS][4], xb[SETS][4];
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
#pragma unroll
    for (int c = 0; c < 4; ++c) xa[s][c] = xb[s][c] = 0.f;
    const T* src = row + (int64_t)min(h0 + s * HPS + sub, heads - 1) * d;
    if (ok) {
      load4(src + j, xa[s]);
      load4(src + j + half, xb[s]);
    }
  }
  float wqa[4] = {1.f, 1.f, 1.f, 1.f}, wqb[4] = {1.f, 1.f, 1.f, 1.f}, wka[4] = {1.f, 1.f, 1.f, 1.f},
        wkb[4] = {1.f, 1.f, 1.f, 1.f};
  if (ok && qw) {
    load4(qw + j, wqa);
    load4(qw + j + half, wqb);
  }
  if (ok && kw) {
    load4(kw + j, wka);
    load4(kw + j + half, wkb);
  }
  pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
  float cv[4] = {1.f, 1.f, 1.f, 1.f}, sv[4] = {0.f, 0.f, 0.f, 0.f};
  if (ok && cos_sin) {
    const float* cs = cos_sin + (int64_t)pos * d;
    load4(cs + j, cv);
    load4(cs + half + j, sv);
  }
  const int P = 1 << page_shift;
#pragma unroll
  for (int s = 0; s < SETS; ++s) {
    const int h = h0 + s * HPS + sub;
    const bool live = h < heads;
    const bool is_key = h >= nq;
    const float* w = is_key ? kw : qw;
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) ss += xa[s][c] * xa[s][c] + xb[s][c] * xb[s][c];
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, MI_WAVE);   // over the head's lanes
    const float rstd = w ? rsqrtf(ss / (float)d + eps) : 1.f;
    float o1[4], o2[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const float a = xa[s][c] * rstd * (is_key ? wka[c] : wqa[c]);
      const float b2 = xb[s][c] * rstd * (is_key ? wkb[c] : wqb[c]);
      o1[c] = a * cv[c] - b2 * sv[c];
      o2[c] = b2 * cv[c] + a * sv[c];
    }
    if (ok && live) {
      T* src = row + (int64_t)h * d;
      store4(src + j, o1);
      store4(src + j + half, o2);
      if (is_key && k_pages) {
        T* dst = k_pages + ((((int64_t)(slot >> page_shift)) * nkv + (h - nq)) * P + (slot & (P - 1))) * d;
        store4(dst + j, o1);
        store4(dst + j + half, o2);
      }
    }
  }
}

// The values of many tokens into their transposed pages [page][kv head][dim][slot in page].  A workgroup takes 16
// consecutive tokens of one kv head.  Consecutive tokens of a request lie side by side in a page, so 16 tokens whose
// slots are consecutive and start at a multiple of 16 are written as one run of 16 per dim (a page's whole row when
// it holds 16 slots), and otherwise each half of 8 tokens whose slots are consecutive and start at a multiple of 8 as
// a run of 8 (16 bytes in bfloat16) instead of scattered elements; any other half falls back to single elements.
template <typename T, int RUN>
__device__ __forceinline__ void value_run_write(const T* __restrict__ src, int64_t row_stride, T* __restrict__ base,
                                                int d, int P) {
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  constexpr int WORDS = RUN * (int)sizeof(T) / 4;
  for (int e = threadIdx.x; e < d; e += blockDim.x) {
    union {
      T v[RUN];
      uint32_t u[WORDS];
    } pack;
#pragma unroll
    for (int i = 0; i < RUN; ++i) pack.v[i] = src[(int64_t)i * row_stride + e];
    uint32_t* o = reinterpret_cast<uint32_t*>(base + (int64_t)e * P);
#pragma unroll
    for (int i = 0; i < WORDS; i += 4)
      *reinterpret_cast<u32x4*>(o + i) = u32x4{pack.u[i], pack.u[i + 1], pack.u[i + 2], pack.u[i + 3]};
  }
}

template <typename T>
__device__ __forceinline__ void value_cache_write_body(int block_x, int g, const T* __restrict__ qkv,
                                                       int64_t row_stride, int nq, int nkv, int d,
                                                       T* __restrict__ v_pages, const int* __restrict__ slots,
                                                       int page_shift, int num_tokens) {
  const int P = 1 << page_shift;
  const int first = block_x * 16;
  if (num_tokens - first >= 16 && P >= 16) {
    const int slot0 = slots[first];
    bool run = (slot0 & 15) == 0;
    for (int i = 1; i < 16; ++i) run = run && slots[first + i] == slot0 + i;
    if (run) {      // the same for every thread of the workgroup
      value_run_write<T, 16>(qkv + (int64_t)first * row_stride + (int64_t)(nq + nkv + g) * d, row_stride,
                             v_pages + (((int64_t)(slot0 >> page_shift) * nkv + g) * d) * P + (slot0 & (P - 1)), d, P);
      return;
    }
  }
  for (int hf = 0; hf < 2; ++hf) {
    const int t0 = first + 8 * hf;
    const int n = min(8, num_tokens - t0);
    if (n <= 0) break;
    const int slot0 = slots[t0];
    bool run = n == 8 && P >= 8 && (slot0 & 7) == 0;
    for (int i = 1; i < n; ++i) run = run && slots[t0 + i] == slot0 + i;
    const T* src = qkv + (int64_t)t0 * row_stride + (int64_t)(nq + nkv + g) * d;
    if (run) {      // the same for every thread of the workgroup
      value_run_write<T, 8>(src, row_stride,
                            v_pages + (((int64_t)(slot0 >> page_shift) * nkv + g) * d) * P + (slot0 & (P - 1)), d, P);
    } else {
      for (int idx = threadIdx.x; idx < n * d; idx += blockDim.x) {
        const int i = idx / d, e = idx - i * d;
        const int slot = slots[t0 + i];
        v_pages[(((int64_t)(slot >> page_shift) * nkv + g) * d + e) * P + (slot & (P - 1))] =
            src[(int64_t)i * row_stride + e];
      }
    }
  }
}

template <typename T, int LPH>
__global__ void qk_norm_rope_many_kernel(T* __restrict__ qkv, int64_t row_stride, int nq, int nkv, int d,
                                         const float* __restrict__ qw, const float* __restrict__ kw, float eps,
                                         const float* __restrict__ cos_sin, int max_pos,
                                         const int* __restrict__ positions, T* __restrict__ k_pages,
                                         const int* __restrict__ slots, int page_shift, int num_tokens) {
  qk_norm_rope_many_body<T, LPH>(blockIdx.x, qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, max_pos, positions,
                                 k_pages, slots, page_shift, num_tokens);
}

// Both at once, for many tokens: the first `norm_blocks` workgroups norm and rotate the q and k heads (and write the
// keys), the others copy the values (workgroup norm_blocks + x + value_blocks_x * g takes tokens 16 x .. of kv head
// g).  The two halves read different columns of qkv and depend on nothing of each other, so one launch does for
// what two launches in a row would wait for each other.
template <typename T, int LPH>
__global__ void qk_norm_rope_values_kernel(T* __restrict__ qkv, int64_t row_stride, int nq, int nkv, int d,
                                           const float* __restrict__ qw, const float* __restrict__ kw, float eps,
                                           const float* __restrict__ cos_sin, int max_pos,
                                           const int* __restrict__ positions, T* __restrict__ k_pages,
                                           T* __restrict__ v_pages, const int* __restrict__ slots, int page_shift,
                                           int num_tokens, int norm_blocks, int value_blocks_x) {
  if ((int)blockIdx.x < norm_blocks) {
    qk_norm_rope_many_body<T, LPH>(blockIdx.x, qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, max_pos, positions,
                                   k_pages, slots, page_shift, num_tokens);
  } else {
    const int b = blockIdx.x - norm_blocks;
    value_cache_write_body<T>(b % value_blocks_x, b / value_blocks_x, qkv, row_stride, nq, nkv, d, v_pages, slots,
                              page_shift, num_tokens);
  }
}

template <typename T>
__global__ void value_cache_write_kernel(const T* __restrict__ qkv, int64_t row_stride, int nq, int nkv, int d,
                                         T* __restrict__ v_pages, const int* __restrict__ slots, int page_shift,
                                         int num_tokens) {
  value_cache_write_body<T>(blockIdx.x, blockIdx.y, qkv, row_stride, nq, nkv, d, v_pages, slots, page_shift,
                            num_tokens);
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
  // many tokens: the values are copied by a kernel of their own that writes runs of slots
  const bool split_values = v_pages && nkv > 0 && num_tokens >= 32 && page_size >= 8;
  const int heads = split_values ? nq + nkv : nq + 2 * nkv;
  const int64_t waves = (int64_t)num_tokens * heads;
  const int blocks = (int)((waves + waves_per_block - 1) / waves_per_block);
  const dim3 vgrid((num_tokens + 15) / 16, nkv > 0 ? nkv : 1);
  const int vthreads = d >= 128 ? 128 : 64;
  // whole-head rotation of many tokens: LPH lanes per head, the power of two >= d / 8
  // (a lane's accesses of 4 elements need the projection and the key pages on multiples of 8 bytes in bfloat16, of
  // 16 in 32-bit, and the 32-bit weights and angles on multiples of 16; anything else goes to the kernel that reads
  // single elements.  8 elements a lane, 16 bytes in bfloat16, were measured and are no quicker: 12.4 against
  // 11.7 us for 2,048 tokens)
  const size_t esz = dtype == MI_DTYPE_F32 ? 4 : 2;
  const bool data_ok = (((uintptr_t)qkv | (uintptr_t)k_pages | (uintptr_t)((size_t)row_stride * esz)) % (4 * esz)) == 0;
  const bool tables_ok = (((uintptr_t)qw | (uintptr_t)kw | (uintptr_t)cos_sin) % 16) == 0;
  const bool many = (split_values || (nkv == 0 && num_tokens >= 32)) && d % 8 == 0 && (!cos_sin || rotary_dim == d) &&
                    data_ok && tables_ok;
  int lph = 1;
  while (lph * 8 < d) lph <<= 1;
  const int heads_per_wave = 2 * (MI_WAVE / lph);
  const int64_t many_waves = (int64_t)num_tokens * ((nq + nkv + heads_per_wave - 1) / heads_per_wave);
  const int many_blocks = (int)((many_waves + waves_per_block - 1) / waves_per_block);
  // many tokens with their values: one launch for both halves
  const bool both = many && split_values;
  const int64_t all_blocks = (int64_t)many_blocks + (int64_t)vgrid.x * vgrid.y;
  MI_REQUIRE(!both || all_blocks < (1ll << 31), "qk_norm_rope_cache: too many workgroups");
#define MI_LAUNCH_MANY(T, LPH)                                                                                      \
  if (both)                                                                                                         \
    qk_norm_rope_values_kernel<T, LPH><<<(unsigned)all_blocks, waves_per_block * MI_WAVE, 0, stream>>>(             \
        (T*)qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, max_pos, positions, (T*)k_pages, (T*)v_pages, slots, \
        shift, num_tokens, many_blocks, (int)vgrid.x);                                                              \
  else                                                                                                              \
    qk_norm_rope_many_kernel<T, LPH><<<many_blocks, waves_per_block * MI_WAVE, 0, stream>>>(                        \
        (T*)qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, max_pos, positions, (T*)k_pages, slots, shift,       \
        num_tokens)
#define MI_LAUNCH_MANY_ANY(T)                                                                                       \
  switch (lph) {                                                                                                    \
    case 1: case 2: MI_LAUNCH_MANY(T, 2); break;                                                                    \
    case 4: MI_LAUNCH_MANY(T, 4); break;                                                                            \
    case 8: MI_LAUNCH_MANY(T, 8); break;                                                                            \
    case 16: MI_LAUNCH_MANY(T, 16); break;                                                                          \
    default: MI_LAUNCH_MANY(T, 32); break;                                                                          \
  }
  if (dtype == MI_DTYPE_F32) {
    if (many) {
      MI_LAUNCH_MANY_ANY(float)
    } else {
      qk_norm_rope_cache_kernel<float><<<blocks, waves_per_block * MI_WAVE, 0, stream>>>(
          (float*)qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, rotary_dim, max_pos, positions, (float*)k_pages,
          (float*)v_pages, slots, shift, num_tokens, heads);
    }
    if (split_values && !both)
      value_cache_write_kernel<float><<<vgrid, vthreads, 0, stream>>>((const float*)qkv, row_stride, nq, nkv, d,
                                                                      (float*)v_pages, slots, shift, num_tokens);
  } else if (dtype == MI_DTYPE_BF16) {
    if (many) {
      MI_LAUNCH_MANY_ANY(bf16)
    } else {
      qk_norm_rope_cache_kernel<bf16><<<blocks, waves_per_block * MI_WAVE, 0, stream>>>(
          (bf16*)qkv, row_stride, nq, nkv, d, qw, kw, eps, cos_sin, rotary_dim, max_pos, positions, (bf16*)k_pages,
          (bf16*)v_pages, slots, shift, num_tokens, heads);
    }
    if (split_values && !both)
      value_cache_write_kernel<bf16><<<vgrid, vthreads, 0, stream>>>((const bf16*)qkv, row_stride, nq, nkv, d,
                                                                     (bf16*)v_pages, slots, shift, num_tokens);
  } else {
    MI_FAIL("qk_norm_rope_cache: unknown dtype %d", dtype);
  }
#undef MI_LAUNCH_MANY_ANY
#undef MI_LAUNCH_MANY
  MI_CHECK_LAUNCH("qk_norm_rope_cache");
  return 0;
}
