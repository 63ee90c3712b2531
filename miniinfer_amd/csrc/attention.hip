// Causal grouped-query attention over a paged cache, any dtype, any head size that is a
// multiple of 8 up to 256, any number of new tokens per request (prompt portions and single
// decoded tokens in one launch).  32-bit scores, softmax and accumulation, no matrix
// instruction: this is the attention of the true 32-bit path and the any-shape fallback of
// the bfloat16 path.
//
// For request b with q_len new tokens and kv_len keys after this step, new token i sits at
// position p = kv_len - q_len + i and sees keys j with max(0, p - window + 1) <= j <= p
// (window 0 = all): the bottom-right aligned causal mask of
// miniinfer/layers/attention.py:112-128; query head h reads kv head h / (nq / nkv)
// (miniinfer/layers/attention.py:131-191); softmax(scale * q.k) v.
//
// One wave per (token, query head).  A tile is 64 keys: each lane scores one key (the query
// is broadcast from LDS), the wave reduces max and sum for the running softmax, then the lanes
// switch to output columns and add the tile's probability-weighted value rows.  With few tokens
// and many keys the key range of each (token, head) is cut into num_splits parts of whole tiles, one
// wave each, which leave an unnormalised sum with its running maximum and denominator in scratch
// memory; a second kernel combines them (the parts' order of summation is the only difference).
// Key pages are [num_pages, nkv, P, d]; value pages are stored transposed, [num_pages, nkv, d, P].
#include "common.h"

template <typename T, int VEC>
__device__ __forceinline__ float dot_row(const float* __restrict__ qs, const T* __restrict__ row, int d);

template <>
__device__ __forceinline__ float dot_row<float, 4>(const float* __restrict__ qs, const float* __restrict__ row, int d) {
  float acc = 0.f;
  for (int e = 0; e < d; e += 4) {
    const float4 kv = *reinterpret_cast<const float4*>(row + e);
    acc = fmaf(qs[e], kv.x, acc);
    acc = fmaf(qs[e + 1], kv.y, acc);
    acc = fmaf(qs[e + 2], kv.z, acc);
    acc = fmaf(qs[e + 3], kv.w, acc);
  }
  return acc;
}

template <>
__device__ __forceinline__ float dot_row<bf16, 8>(const float* __restrict__ qs, const bf16* __restrict__ row, int d) {
  float acc = 0.f;
  for (int e = 0; e < d; e += 8) {
    const uint4 raw = *reinterpret_cast<const uint4*>(row + e);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc = fmaf(qs[e + 2 * i], __uint_as_float(w[i] << 16), acc);
      acc = fmaf(qs[e + 2 * i + 1], __uint_as_float(w[i] & 0xffff0000u), acc);
    }
  }
  return acc;
}

template <typename T, int VEC>
__global__ __launch_bounds__(256) void paged_attention_kernel(
    const T* __restrict__ q, int64_t q_row_stride, T* __restrict__ out, int64_t out_row_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ token_req, const int* __restrict__ cu_q, const int* __restrict__ kv_len, int num_tokens,
    int nq, int nkv, int d, int page_shift, float scale, int window, int num_splits, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  extern __shared__ float smem[];
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int wave = threadIdx.x / MI_WAVE;
  float* qs = smem + wave * d;
  const int64_t wid = (int64_t)blockIdx.x * (blockDim.x / MI_WAVE) + wave;
  const bool live = wid < (int64_t)num_tokens * nq * num_splits;
  int t = 0, h = 0, split = 0;
  if (live) {
    const int64_t th = wid / num_splits;
    split = (int)(wid - th * num_splits);
    t = (int)(th / nq);
    h = (int)(th - (int64_t)t * nq);
    const T* qr = q + (int64_t)t * q_row_stride + (int64_t)h * d;
    for (int e = lane; e < d; e += MI_WAVE) qs[e] = to_float(qr[e]);
  }
  __syncthreads();
  if (!live) return;

  const int b = token_req[t];
  const int q_begin = cu_q[b];
  const int q_len = cu_q[b + 1] - q_begin;
  const int pos = kv_len[b] - q_len + (t - q_begin);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int g = h / (nq / nkv);
  const int P = 1 << page_shift;
  const int* bt = block_table + (int64_t)b * table_width;

  // this wave's part of the tiles of lo .. pos (the first part is never empty)
  const int tiles = (pos - lo) / MI_WAVE + 1;
  const int tiles_per_split = (tiles + num_splits - 1) / num_splits;
  const int j_begin = lo + split * tiles_per_split * MI_WAVE;
  const int j_stop = (split + 1 == num_splits) ? pos + 1 : min(pos + 1, j_begin + tiles_per_split * MI_WAVE);

  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};

  for (int j0 = j_begin; j0 < j_stop; j0 += MI_WAVE) {
    const int j = j0 + lane;
    float s = -INFINITY;
    if (j <= pos) {
      const int64_t page = bt[j >> page_shift];
      const T* row = k_pages + ((page * nkv + g) * P + (j & (P - 1))) * d;
      s = dot_row<T, VEC>(qs, row, d) * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));   // the tile's first key is visible, so m_new is finite
    const float p = (j <= pos) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);         // 0 on the first tile (m = -inf)
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[c] *= alpha;
    const int n = (pos - j0 + 1 < MI_WAVE) ? pos - j0 + 1 : MI_WAVE;
    for (int i = 0; i < n; ++i) {
      const float pi = __shfl(p, i, MI_WAVE);
      const int jj = j0 + i;
      const int64_t page = bt[jj >> page_shift];
      const T* vcol = v_pages + (page * nkv + g) * (int64_t)d * P + (jj & (P - 1));   // value pages are [d][P]
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = lane + c * MI_WAVE;
        if (e < d) acc[c] = fmaf(pi, to_float(vcol[(int64_t)e * P]), acc[c]);
      }
    }
  }
  if (num_splits > 1) {
    float* po = part_o + wid * d;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e = lane + c * MI_WAVE;
      if (e < d) po[e] = acc[c];
    }
    if (lane == 0) {
      part_ml[wid * 2] = m;
      part_ml[wid * 2 + 1] = l;
    }
    return;
  }
  T* o = out + (int64_t)t * out_row_stride + (int64_t)h * d;
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int e = lane + c * MI_WAVE;
    if (e < d) o[e] = from_float<T>(acc[c] * inv);
  }
}

// One wave per (token, head): out = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s with M = max_s m_s.
// An empty part has m = -inf and l = 0 and adds nothing; the first part is never empty, so M is finite.
template <typename T>
__global__ __launch_bounds__(256) void paged_attention_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, T* __restrict__ out, int64_t out_row_stride,
    int num_tokens, int nq, int d, int num_splits) {
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int64_t th = (int64_t)blockIdx.x * (blockDim.x / MI_WAVE) + threadIdx.x / MI_WAVE;
  if (th >= (int64_t)num_tokens * nq) return;
  const float* ml = part_ml + th * num_splits * 2;
  float M = -INFINITY;
  for (int s = 0; s < num_splits; ++s) M = fmaxf(M, ml[2 * s]);
  float l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int s = 0; s < num_splits; ++s) {
    const float w = expf(ml[2 * s] - M);
    l = fmaf(w, ml[2 * s + 1], l);
    const float* po = part_o + (th * num_splits + s) * d;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int e = lane + c * MI_WAVE;
      if (e < d) acc[c] = fmaf(w, po[e], acc[c]);
    }
  }
  const int t = (int)(th / nq);
  const int h = (int)(th - (int64_t)t * nq);
  T* o = out + (int64_t)t * out_row_stride + (int64_t)h * d;
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    const int e = lane + c * MI_WAVE;
    if (e < d) o[e] = from_float<T>(acc[c] * inv);
  }
}

MI_EXPORT int mi_paged_attention(int dtype, const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride,
                                 const void* k_pages, const void* v_pages, const int* block_table, int table_width,
                                 const int* token_req, const int* cu_q, const int* kv_len, int num_tokens,
                                 int num_requests, int nq, int nkv, int d, int page_size, float scale, int window,
                                 int num_splits, float* part_o, float* part_ml, hipStream_t stream) {
  MI_REQUIRE(num_tokens >= 0 && num_requests >= 0 && nq > 0 && nkv > 0, "paged_attention: bad sizes");
  MI_REQUIRE(nq % nkv == 0, "paged_attention: %d query heads are no multiple of %d kv heads", nq, nkv);
  MI_REQUIRE(d > 0 && d % 8 == 0 && d <= 256, "paged_attention: head size %d is not a multiple of 8 up to 256", d);
  MI_REQUIRE(page_size > 0 && (page_size & (page_size - 1)) == 0, "paged_attention: page size %d is no power of two",
             page_size);
  MI_REQUIRE(q_row_stride >= (int64_t)nq * d && out_row_stride >= (int64_t)nq * d, "paged_attention: row strides too small");
  MI_REQUIRE(q_row_stride % 8 == 0, "paged_attention: query row stride %lld is not a multiple of 8", (long long)q_row_stride);
  MI_REQUIRE(window >= 0 && table_width > 0, "paged_attention: bad window or table width");
  MI_REQUIRE(num_splits >= 1 && num_splits <= 1024, "paged_attention: %d key parts are not in 1..1024", num_splits);
  MI_REQUIRE(num_splits == 1 || (part_o != nullptr && part_ml != nullptr),
             "paged_attention: key parts need scratch memory for their partial sums");
  if (num_tokens == 0) return 0;
  int shift = 0;
  while ((1 << shift) < page_size) ++shift;
  const int waves_per_block = 4;
  const int64_t waves = (int64_t)num_tokens * nq * num_splits;
  MI_REQUIRE(waves / waves_per_block < (int64_t)INT32_MAX, "paged_attention: too many (token, head, part) items");
  const int blocks = (int)((waves + waves_per_block - 1) / waves_per_block);
  const size_t lds = (size_t)waves_per_block * d * sizeof(float);
  if (dtype == MI_DTYPE_F32)
    paged_attention_kernel<float, 4><<<blocks, waves_per_block * MI_WAVE, lds, stream>>>(
        (const float*)q, q_row_stride, (float*)out, out_row_stride, (const float*)k_pages, (const float*)v_pages,
        block_table, table_width, token_req, cu_q, kv_len, num_tokens, nq, nkv, d, shift, scale, window, num_splits,
        part_o, part_ml);
  else if (dtype == MI_DTYPE_BF16)
    paged_attention_kernel<bf16, 8><<<blocks, waves_per_block * MI_WAVE, lds, stream>>>(
        (const bf16*)q, q_row_stride, (bf16*)out, out_row_stride, (const bf16*)k_pages, (const bf16*)v_pages,
        block_table, table_width, token_req, cu_q, kv_len, num_tokens, nq, nkv, d, shift, scale, window, num_splits,
        part_o, part_ml);
  else
    MI_FAIL("paged_attention: unknown dtype %d", dtype);
  MI_CHECK_LAUNCH("paged_attention");
  if (num_splits > 1) {
    const int merge_blocks = (int)(((int64_t)num_tokens * nq + waves_per_block - 1) / waves_per_block);
    if (dtype == MI_DTYPE_F32)
      paged_attention_merge_kernel<float><<<merge_blocks, waves_per_block * MI_WAVE, 0, stream>>>(
          part_o, part_ml, (float*)out, out_row_stride, num_tokens, nq, d, num_splits);
    else
      paged_attention_merge_kernel<bf16><<<merge_blocks, waves_per_block * MI_WAVE, 0, stream>>>(
          part_o, part_ml, (bf16*)out, out_row_stride, num_tokens, nq, d, num_splits);
    MI_CHECK_LAUNCH("paged_attention_merge");
  }
  return 0;
}
