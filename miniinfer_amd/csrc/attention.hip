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
// One wave per (token, query heads of one kv head).  A tile is 64 keys: each lane scores one key against the
// wave's queries (broadcast from LDS; the key row is loaded once for all of them), the wave reduces max and sum
// for each head's running softmax, then the lanes switch to output columns and add the tile's probability-weighted
// value rows.  With few tokens and many keys the key range of each token is cut into num_splits parts of whole
// tiles, one wave each, which leave an unnormalised sum with its running maximum and denominator in scratch
// memory; a second kernel combines them (the parts' order of summation is the only difference).
// Key pages are [num_pages, nkv, P, d]; value pages are stored transposed, [num_pages, nkv, d, P].
#include "common.h"

// scores of one key row against REP queries (qs [REP][d] in LDS): every element of the row is loaded once; each
// query's sum is one chain of fused multiply-adds over the dims in ascending order
template <typename T, int REP>
__device__ __forceinline__ void dot_rows(const float* __restrict__ qs, const T* __restrict__ row, int d, float (&s)[REP]);

template <int REP>
__device__ __forceinline__ void dot_rows_f32(const float* __restrict__ qs, const float* __restrict__ row, int d, float (&s)[REP]) {
#pragma unroll
  for (int x = 0; x < REP; ++x) s[x] = 0.f;
#pragma unroll 4
  for (int e = 0; e < d; e += 4) {
    float kv[4];
    load4(row + e, kv);
#pragma unroll
    for (int x = 0; x < REP; ++x)
#pragma unroll
      for (int i = 0; i < 4; ++i) s[x] = fmaf(qs[x * d + e + i], kv[i], s[x]);
  }
}

template <int REP>
__device__ __forceinline__ void dot_rows_bf16(const float* __restrict__ qs, const bf16* __restrict__ row, int d, float (&s)[REP]) {
#pragma unroll
  for (int x = 0; x < REP; ++x) s[x] = 0.f;
#pragma unroll 2
  for (int e = 0; e < d; e += 8) {
    float kv[8];
    load4(row + e, *reinterpret_cast<float(*)[4]>(&kv[0]));
    load4(row + e + 4, *reinterpret_cast<float(*)[4]>(&kv[4]));
#pragma unroll
    for (int x = 0; x < REP; ++x)
#pragma unroll
      for (int i = 0; i < 8; ++i) s[x] = fmaf(qs[x * d + e + i], kv[i], s[x]);
  }
}

template <int REP>
__device__ __forceinline__ void dot_rows_any(const float* qs, const float* row, int d, float (&s)[REP]) { dot_rows_f32<REP>(qs, row, d, s); }
template <int REP>
__device__ __forceinline__ void dot_rows_any(const float* qs, const bf16* row, int d, float (&s)[REP]) { dot_rows_bf16<REP>(qs, row, d, s); }

// One wave per (token, group of REP query heads, key range).  REP = the query heads of a kv head when that is 1, 2, 4
// or 8 (the keys and values are then read once for all of them), else 1 (a wave per query head).
template <typename T, int REP>
__global__ __launch_bounds__(256) void paged_attention_kernel(
    const T* __restrict__ q, int64_t q_row_stride, T* __restrict__ out, int64_t out_row_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ token_req, const int* __restrict__ cu_q, const int* __restrict__ kv_len, int num_tokens,
    int nq, int nkv, int d, int page_shift, float scale, int window, int num_splits, float* __restrict__ part_o,
    float* __restrict__ part_ml) {
  extern __shared__ float smem[];
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int wave = threadIdx.x / MI_WAVE;
  float* qs = smem + wave * REP * d;
  const int groups = nq / REP;               // head groups per token
  const int64_t wid = (int64_t)blockIdx.x * (blockDim.x / MI_WAVE) + wave;
  const bool live = wid < (int64_t)num_tokens * groups * num_splits;
  int t = 0, h0 = 0, split = 0;
  if (live) {
    const int64_t tg = wid / num_splits;
    split = (int)(wid - tg * num_splits);
    t = (int)(tg / groups);
    h0 = (int)(tg - (int64_t)t * groups) * REP;
    const T* qr = q + (int64_t)t * q_row_stride + (int64_t)h0 * d;
    for (int e = lane; e < REP * d; e += MI_WAVE) qs[e] = to_float(qr[e]);
  }
  __syncthreads();
  if (!live) return;

  const int b = token_req[t];
  const int q_begin = cu_q[b];
  const int q_len = cu_q[b + 1] - q_begin;
  const int pos = kv_len[b] - q_len + (t - q_begin);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int g = h0 / (nq / nkv);
  const int P = 1 << page_shift;
  const int* bt = block_table + (int64_t)b * table_width;

  // this wave's part of the tiles of lo .. pos: the tiles are shared out evenly, the parts differ by one tile at
  // most (with fewer tiles than parts some parts are empty; they leave m = -inf, l = 0)
  const int tiles = (pos - lo) / MI_WAVE + 1;
  const int j_begin = lo + (int)((int64_t)split * tiles / num_splits) * MI_WAVE;
  const int j_stop = (split + 1 == num_splits) ? pos + 1 : lo + (int)((int64_t)(split + 1) * tiles / num_splits) * MI_WAVE;

  float m[REP], l[REP], acc[REP][4];
#pragma unroll
  for (int x = 0; x < REP; ++x) {
    m[x] = -INFINITY;
    l[x] = 0.f;
#pragma unroll
    for (int c = 0; c < 4; ++c) acc[x][c] = 0.f;
  }

  for (int j0 = j_begin; j0 < j_stop; j0 += MI_WAVE) {
    const int j = j0 + lane;
    float s[REP], p[REP];
#pragma unroll
    for (int x = 0; x < REP; ++x) s[x] = -INFINITY;
    if (j <= pos) {
      const int64_t page = bt[j >> page_shift];
      const T* row = k_pages + ((page * nkv + g) * P + (j & (P - 1))) * d;
      dot_rows_any<REP>(qs, row, d, s);
#pragma unroll
      for (int x = 0; x < REP; ++x) s[x] *= scale;
    }
#pragma unroll
    for (int x = 0; x < REP; ++x) {
      const float m_new = fmaxf(m[x], wave_max(s[x]));   // the tile's first key is visible, so m_new is finite
      p[x] = (j <= pos) ? expf(s[x] - m_new) : 0.f;
      const float alpha = expf(m[x] - m_new);            // 0 on the first tile (m = -inf)
      l[x] = l[x] * alpha + wave_sum(p[x]);
      m[x] = m_new;
#pragma unroll
      for (int c = 0; c < 4; ++c) acc[x][c] *= alpha;
    }
    // The tile's value rows, page by page: in the transposed pages [d][P] the keys of a page lie side by side for
    // every dim, so a lane reads runs of 4 keys of its dims at once (where the page and the run allow it) and looks
    // the page up once.  The products are added key by key in ascending order either way.
    const int n = (pos - j0 + 1 < MI_WAVE) ? pos - j0 + 1 : MI_WAVE;
    for (int i = 0; i < n;) {
      const int jj = j0 + i;
      const int in_page = jj & (P - 1);
      const int run = min(n - i, P - in_page);
      const int64_t page = bt[jj >> page_shift];
      const T* vbase = v_pages + (page * nkv + g) * (int64_t)d * P + in_page;
      for (int u = 0; u < run;) {
        if (P >= 4 && ((in_page + u) & 3) == 0 && u + 4 <= run) {
          float pk[REP][4];
#pragma unroll
          for (int x = 0; x < REP; ++x)
#pragma unroll
            for (int y = 0; y < 4; ++y) pk[x][y] = __shfl(p[x], i + u + y, MI_WAVE);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int e = lane + c * MI_WAVE;
            if (e < d) {
              float v4[4];
              load4(vbase + (int64_t)e * P + u, v4);
#pragma unroll
              for (int x = 0; x < REP; ++x)
#pragma unroll
                for (int y = 0; y < 4; ++y) acc[x][c] = fmaf(pk[x][y], v4[y], acc[x][c]);
            }
          }
          u += 4;
        } else {
          float pi[REP];
#pragma unroll
          for (int x = 0; x < REP; ++x) pi[x] = __shfl(p[x], i + u, MI_WAVE);
#pragma unroll
          for (int c = 0; c < 4; ++c) {
            const int e = lane + c * MI_WAVE;
            if (e < d) {
              const float vv = to_float(vbase[(int64_t)e * P + u]);
#pragma unroll
              for (int x = 0; x < REP; ++x) acc[x][c] = fmaf(pi[x], vv, acc[x][c]);
            }
          }
          u += 1;
        }
      }
      i += run;
    }
  }
#pragma unroll
  for (int x = 0; x < REP; ++x) {
    const int h = h0 + x;
    if (num_splits > 1) {
      const int64_t item = ((int64_t)t * nq + h) * num_splits + split;
      float* po = part_o + item * d;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = lane + c * MI_WAVE;
        if (e < d) po[e] = acc[x][c];
      }
      if (lane == 0) {
        part_ml[item * 2] = m[x];
        part_ml[item * 2 + 1] = l[x];
      }
    } else {
      T* o = out + (int64_t)t * out_row_stride + (int64_t)h * d;
      const float inv = 1.f / l[x];
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int e = lane + c * MI_WAVE;
        if (e < d) o[e] = from_float<T>(acc[x][c] * inv);
      }
    }
  }
}

// The same wave per (token, query heads of one kv head, key range) for 32-bit caches with head sizes in steps of 16
// up to 128 and pages of 16 keys or more, with every load instruction of the wave covering whole lines of memory:
// four lanes share a key.  Scores: lane (key = lane / 4, quarter = lane % 4) reads floats 16 i + 4 quarter .. + 3 of
// its key's row for every i, so the four lanes read 64 bytes side by side and the wave 16 keys at a time; each lane's
// partial score is one chain of fused multiply-adds over its dims in ascending order, the four are added as
// (0 + 1) + (2 + 3), and four such passes give the tile's 64 scores, which are then moved to one key a lane.
// Values: in the transposed pages a dim's 16 keys of a block are 64 bytes; lane (dim = lane / 4 + 16 c, quarter)
// reads keys 4 quarter .. + 3 of the block and keeps its own sum for the dim, keys ascending; the four quarters' sums
// are added once, at the end.  Blocks of 16 keys are aligned in the pages, so a tile that does not start on one (a
// window's edge) and the last tile take their ragged blocks key by key.
// DC = head size / 16 is a parameter of the build (64, 80, 96 and 128 are built), so that no branch stands between a
// tile's loads.
template <int REP, int DC>
__global__ __launch_bounds__(256) void paged_attention_quad_kernel(
    const float* __restrict__ q, int64_t q_row_stride, float* __restrict__ out, int64_t out_row_stride,
    const float* __restrict__ k_pages, const float* __restrict__ v_pages, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ token_req, const int* __restrict__ cu_q, const int* __restrict__ kv_len,
    int num_tokens, int nq, int nkv, int d, int page_shift, float scale, int window, int num_splits,
    float* __restrict__ part_o, float* __restrict__ part_ml) {
  extern __shared__ float smem[];
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int wave = threadIdx.x / MI_WAVE;
  float* qs = smem + wave * REP * d;
  const int groups = nq / REP;
  const int64_t wid = (int64_t)blockIdx.x * (blockDim.x / MI_WAVE) + wave;
  const bool live = wid < (int64_t)num_tokens * groups * num_splits;
  int t = 0, h0 = 0, split = 0;
  if (live) {
    const int64_t tg = wid / num_splits;
    split = (int)(wid - tg * num_splits);
    t = (int)(tg / groups);
    h0 = (int)(tg - (int64_t)t * groups) * REP;
    const float* qr = q + (int64_t)t * q_row_stride + (int64_t)h0 * d;
    for (int e = lane; e < REP * d; e += MI_WAVE) qs[e] = qr[e];
  }
  __syncthreads();
  if (!live) return;

  const int b = token_req[t];
  const int q_begin = cu_q[b];
  const int q_len = cu_q[b + 1] - q_begin;
  const int pos = kv_len[b] - q_len + (t - q_begin);
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int g = h0 / (nq / nkv);
  const int P = 1 << page_shift;
  const int* bt = block_table + (int64_t)b * table_width;
  const int quad = lane >> 2, quarter = lane & 3;

  const int tiles = (pos - lo) / MI_WAVE + 1;
  const int j_begin = lo + (int)((int64_t)split * tiles / num_splits) * MI_WAVE;
  const int j_stop = (split + 1 == num_splits) ? pos + 1 : lo + (int)((int64_t)(split + 1) * tiles / num_splits) * MI_WAVE;

  float m[REP], l[REP], acc[REP][DC];
#pragma unroll
  for (int x = 0; x < REP; ++x) {
    m[x] = -INFINITY;
    l[x] = 0.f;
#pragma unroll
    for (int c = 0; c < DC; ++c) acc[x][c] = 0.f;
  }

  for (int j0 = j_begin; j0 < j_stop; j0 += MI_WAVE) {
    // scores: four passes of 16 keys; a key past pos reads the row of pos and is masked below
    float sc[4][REP];
#pragma unroll        // all four passes' loads on their way together (one or two at a time: 39 against 31.5 us)
    for (int pass = 0; pass < 4; ++pass) {
      const int jk = min(j0 + pass * 16 + quad, pos);
      const int64_t page = bt[jk >> page_shift];
      const float* row = k_pages + ((page * nkv + g) * P + (jk & (P - 1))) * d + 4 * quarter;
#pragma unroll
      for (int x = 0; x < REP; ++x) sc[pass][x] = 0.f;
#pragma unroll
      for (int i = 0; i < DC; ++i) {
        float kv[4];
        load4(row + 16 * i, kv);
#pragma unroll
        for (int x = 0; x < REP; ++x) {
          float qv[4];
          load4(qs + x * d + 16 * i + 4 * quarter, qv);
#pragma unroll
          for (int y = 0; y < 4; ++y) sc[pass][x] = fmaf(qv[y], kv[y], sc[pass][x]);
        }
      }
#pragma unroll
      for (int x = 0; x < REP; ++x) {
        sc[pass][x] += __shfl_xor(sc[pass][x], 1, MI_WAVE);
        sc[pass][x] += __shfl_xor(sc[pass][x], 2, MI_WAVE);
      }
    }
    // one key a lane: lane L takes key j0 + L, which pass L / 16 left in the lanes of quad L % 16
    const int j = j0 + lane;
    float s[REP], p[REP];
#pragma unroll
    for (int x = 0; x < REP; ++x) {
      const int src = 4 * (lane & 15);
      const float s0 = __shfl(sc[0][x], src, MI_WAVE), s1 = __shfl(sc[1][x], src, MI_WAVE);
      const float s2 = __shfl(sc[2][x], src, MI_WAVE), s3 = __shfl(sc[3][x], src, MI_WAVE);
      const int pass = lane >> 4;
      const float v = pass == 0 ? s0 : (pass == 1 ? s1 : (pass == 2 ? s2 : s3));
      s[x] = (j <= pos) ? v * scale : -INFINITY;
    }
#pragma unroll
    for (int x = 0; x < REP; ++x) {
      const float m_new = fmaxf(m[x], wave_max(s[x]));
      p[x] = (j <= pos) ? expf(s[x] - m_new) : 0.f;
      const float alpha = expf(m[x] - m_new);
      l[x] = l[x] * alpha + wave_sum(p[x]);
      m[x] = m_new;
#pragma unroll
      for (int c = 0; c < DC; ++c) acc[x][c] *= alpha;
    }
    // values: the aligned blocks of 16 keys that hold keys j0 .. j_end - 1
    const int j_end = min(j0 + MI_WAVE, pos + 1);
    for (int bs = j0 & ~15; bs < j_end; bs += 16) {
      const int64_t page = bt[bs >> page_shift];
      const float* vbase = v_pages + (page * nkv + g) * (int64_t)d * P + (bs & (P - 1)) + 4 * quarter;
      const int k0 = bs + 4 * quarter;           // this lane's four keys of the block
      if (bs >= j0 && bs + 16 <= j_end) {
        float pk[REP][4];
#pragma unroll
        for (int x = 0; x < REP; ++x)
#pragma unroll
          for (int y = 0; y < 4; ++y) pk[x][y] = __shfl(p[x], k0 - j0 + y, MI_WAVE);
#pragma unroll
        for (int c = 0; c < DC; ++c) {
          float v4[4];
          load4(vbase + (int64_t)(quad + 16 * c) * P, v4);
#pragma unroll
          for (int x = 0; x < REP; ++x)
#pragma unroll
            for (int y = 0; y < 4; ++y) acc[x][c] = fmaf(pk[x][y], v4[y], acc[x][c]);
        }
      } else {
#pragma unroll
        for (int y = 0; y < 4; ++y) {
          const int key = k0 + y;
          const bool inside = key >= j0 && key < j_end;
          float pk[REP];
#pragma unroll
          for (int x = 0; x < REP; ++x) pk[x] = __shfl(p[x], inside ? key - j0 : 0, MI_WAVE);
          if (inside) {
#pragma unroll
            for (int c = 0; c < DC; ++c) {
              const float vv = vbase[(int64_t)(quad + 16 * c) * P + y];
#pragma unroll
              for (int x = 0; x < REP; ++x) acc[x][c] = fmaf(pk[x], vv, acc[x][c]);
            }
          }
        }
      }
    }
  }
  // the four quarters' sums of a dim, added as (0 + 1) + (2 + 3); quarter u then stores the dims of blocks c = u mod 4
#pragma unroll
  for (int x = 0; x < REP; ++x) {
#pragma unroll
    for (int c = 0; c < DC; ++c) {
      acc[x][c] += __shfl_xor(acc[x][c], 1, MI_WAVE);
      acc[x][c] += __shfl_xor(acc[x][c], 2, MI_WAVE);
    }
    const int h = h0 + x;
    if (num_splits > 1) {
      const int64_t item = ((int64_t)t * nq + h) * num_splits + split;
      float* po = part_o + item * d;
#pragma unroll
      for (int c = 0; c < DC; ++c)
        if ((c & 3) == quarter) po[quad + 16 * c] = acc[x][c];
      if (lane == 0) {
        part_ml[item * 2] = m[x];
        part_ml[item * 2 + 1] = l[x];
      }
    } else {
      float* o = out + (int64_t)t * out_row_stride + (int64_t)h * d;
      const float inv = 1.f / l[x];
#pragma unroll
      for (int c = 0; c < DC; ++c)
        if ((c & 3) == quarter) o[quad + 16 * c] = acc[x][c] * inv;
    }
  }
}

// One workgroup per (token, head): out = sum_s exp(m_s - M) acc_s / sum_s exp(m_s - M) l_s with M = max_s m_s.
// An empty part has m = -inf and l = 0 and adds nothing; the last part is never empty, so M is finite.
// The parts' weights are made once, by the lanes side by side, and kept in LDS; then thread (group, dim) adds the
// parts group, group + G, ... of its dim (G = 256 / the head size rounded up to a power of two), whose loads do not
// depend on one another, and the groups' sums are added in order.
#define MERGE_THREADS 256
template <typename T>
__global__ __launch_bounds__(MERGE_THREADS) void paged_attention_merge_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, T* __restrict__ out, int64_t out_row_stride,
    int num_tokens, int nq, int d, int dpad, int num_splits) {
  extern __shared__ float msm[];             // [num_splits] weights, [MERGE_THREADS] partial sums, [4] the waves' l
  float* wts = msm;
  float* red = msm + num_splits;
  float* lsum = red + MERGE_THREADS;
  const int tid = threadIdx.x, lane = tid & (MI_WAVE - 1), wave = tid / MI_WAVE;
  const int64_t th = blockIdx.x;
  const float* ml = part_ml + th * num_splits * 2;
  float M = -INFINITY;
  for (int s = tid; s < num_splits; s += MERGE_THREADS) M = fmaxf(M, ml[2 * s]);
  M = wave_max(M);
  if (lane == 0) lsum[wave] = M;
  __syncthreads();
  M = fmaxf(fmaxf(lsum[0], lsum[1]), fmaxf(lsum[2], lsum[3]));
  __syncthreads();
  float l = 0.f;
  for (int s = tid; s < num_splits; s += MERGE_THREADS) {
    const float w = expf(ml[2 * s] - M);
    wts[s] = w;
    l = fmaf(w, ml[2 * s + 1], l);
  }
  l = wave_sum(l);
  if (lane == 0) lsum[wave] = l;
  __syncthreads();
  l = (lsum[0] + lsum[1]) + (lsum[2] + lsum[3]);
  const int G = MERGE_THREADS / dpad;
  const int grp = tid / dpad, e = tid % dpad;
  float acc = 0.f;
  if (e < d) {
    const float* po = part_o + th * num_splits * d + e;
#pragma unroll 8
    for (int s = grp; s < num_splits; s += G) acc = fmaf(wts[s], po[(int64_t)s * d], acc);
  }
  red[tid] = acc;
  __syncthreads();
  if (grp == 0 && e < d) {
    float v = red[e];
    for (int g2 = 1; g2 < G; ++g2) v += red[g2 * dpad + e];
    const int t = (int)(th / nq);
    const int h = (int)(th - (int64_t)t * nq);
    out[(int64_t)t * out_row_stride + (int64_t)h * d + e] = from_float<T>(v / l);
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
  const int per_kv = nq / nkv;
  int rep = (per_kv == 2 || per_kv == 4 || per_kv == 8) ? per_kv : 1;
  // the kernel with four lanes a key: 32-bit, head sizes it is built for, pages of whole blocks of 16 keys; it holds
  // more of a tile in registers, so eight query heads of a kv head go to two waves of four
  const bool quads = dtype == MI_DTYPE_F32 && (d == 64 || d == 80 || d == 96 || d == 128) && page_size >= 16 &&
                     q_row_stride % 4 == 0 && (uintptr_t)q % 16 == 0 && (uintptr_t)k_pages % 16 == 0 &&
                     (uintptr_t)v_pages % 16 == 0;
  if (quads && rep == 8) rep = 4;
  const int64_t waves = (int64_t)num_tokens * (nq / rep) * num_splits;
  MI_REQUIRE(waves / waves_per_block < (int64_t)INT32_MAX, "paged_attention: too many (token, head, part) items");
  const int blocks = (int)((waves + waves_per_block - 1) / waves_per_block);
  const size_t lds = (size_t)waves_per_block * rep * d * sizeof(float);
#define ATTN_GO(T, REP)                                                                                              \
  paged_attention_kernel<T, REP><<<blocks, waves_per_block * MI_WAVE, lds, stream>>>(                               \
      (const T*)q, q_row_stride, (T*)out, out_row_stride, (const T*)k_pages, (const T*)v_pages, block_table,        \
      table_width, token_req, cu_q, kv_len, num_tokens, nq, nkv, d, shift, scale, window, num_splits, part_o, part_ml)
#define ATTN_REP(T)                                                                                                 \
  if (rep == 8) ATTN_GO(T, 8);                                                                                      \
  else if (rep == 4) ATTN_GO(T, 4);                                                                                 \
  else if (rep == 2) ATTN_GO(T, 2);                                                                                 \
  else ATTN_GO(T, 1)
#define ATTN_QUAD(REP, DC)                                                                                           \
  paged_attention_quad_kernel<REP, DC><<<blocks, waves_per_block * MI_WAVE, lds, stream>>>(                         \
      (const float*)q, q_row_stride, (float*)out, out_row_stride, (const float*)k_pages, (const float*)v_pages,     \
      block_table, table_width, token_req, cu_q, kv_len, num_tokens, nq, nkv, d, shift, scale, window, num_splits,  \
      part_o, part_ml)
#define ATTN_QUAD_REP(DC)                                                                                            \
  if (rep == 4) ATTN_QUAD(4, DC);                                                                                    \
  else if (rep == 2) ATTN_QUAD(2, DC);                                                                               \
  else ATTN_QUAD(1, DC)
  if (quads) {
    if (d == 64) { ATTN_QUAD_REP(4); }
    else if (d == 80) { ATTN_QUAD_REP(5); }
    else if (d == 96) { ATTN_QUAD_REP(6); }
    else { ATTN_QUAD_REP(8); }
  } else if (dtype == MI_DTYPE_F32) {
    ATTN_REP(float);
  } else if (dtype == MI_DTYPE_BF16) {
    ATTN_REP(bf16);
  } else
    MI_FAIL("paged_attention: unknown dtype %d", dtype);
#undef ATTN_QUAD_REP
#undef ATTN_QUAD
#undef ATTN_REP
#undef ATTN_GO
  MI_CHECK_LAUNCH("paged_attention");
  if (num_splits > 1) {
    int dpad = 8;
    while (dpad < d) dpad *= 2;
    const int merge_blocks = num_tokens * nq;
    const size_t mlds = ((size_t)num_splits + MERGE_THREADS + 4) * sizeof(float);
    if (dtype == MI_DTYPE_F32)
      paged_attention_merge_kernel<float><<<merge_blocks, MERGE_THREADS, mlds, stream>>>(
          part_o, part_ml, (float*)out, out_row_stride, num_tokens, nq, d, dpad, num_splits);
    else
      paged_attention_merge_kernel<bf16><<<merge_blocks, MERGE_THREADS, mlds, stream>>>(
          part_o, part_ml, (bf16*)out, out_row_stride, num_tokens, nq, d, dpad, num_splits);
    MI_CHECK_LAUNCH("paged_attention_merge");
  }
  return 0;
}
