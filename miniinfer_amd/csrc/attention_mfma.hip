// bfloat16 attention over the paged cache on the matrix cores (MFMA) of gfx950, for one head size
// (compile with -DHEAD_DIM=<multiple of 16, at most 256>).
//
// Same function as attention.hip (bottom-right aligned causal mask, optional window, grouped heads:
// miniinfer/layers/attention.py:112-191), in two launches:
//   prefill: entries with several new tokens; one wave per (kv head, block of query columns);
//   decode:  entries with one new token; the keys of a request are split over several waves
//            (flash-decoding), which write (max, sum, unnormalised output) partials that a merge kernel
//            combines with the log-sum-exp rule.
//
// Layout of the products, chosen so that every operand comes straight from global memory or from the
// previous product's accumulators, with no trip through LDS:
//   S^T[key, col] = K[key, :] . Q[col, :]      A = K rows (16 B per lane from a key's row), B = Q rows
//   O^T[dim, col] = V^T[dim, :] . P^T[:, col]  A = V^T rows (value pages are stored [dim][key in page]),
//                                              B = P, which is exactly where S^T's accumulators sit
// A "column" is a (query token, query head of the kv group) pair; 16 columns form an MFMA block.  All
// softmax statistics of a column live in the lanes with lane % 16 == column.  Scores, softmax and
// accumulation are 32-bit; P is rounded to bfloat16 for the second product.
#include "common.h"

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be a multiple of 16 up to 256");

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int D = HEAD_DIM;
constexpr int KSTEPS = D / 32;          // 16x16x32 products over the head dim
constexpr bool KREM = (D % 32) != 0;    // plus one more, half of it zeros
constexpr int DBLK = D / 16;            // 16-row blocks of O^T

// The last 16 dims of a head size that is no multiple of 32 go through the same 16x16x32 product with the
// upper half of the contraction zeroed: lanes 0..31 hold 8 dims each, lanes 32..63 hold zeros.  (Finishing
// the score with a 16x16x16 product on the accumulator of the 16x16x32 ones gave wrong sums on gfx950 with
// hipcc 7.2 whenever a wave ran more than one tile; one opcode per accumulator chain does not.)
struct QRegs {
  bf16x8 full[KSTEPS + (KREM ? 1 : 0)];
};
constexpr int QSTEPS = KSTEPS + (KREM ? 1 : 0);

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

// operand registers of one row (a key's or a query's `D` elements) in the lane's MFMA slots
__device__ __forceinline__ void load_row(bf16x8 (&r)[QSTEPS], const uint16_t* row, bool ok) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s) {
    r[s] = *reinterpret_cast<const bf16x8*>(row + 32 * s + 8 * (lane >> 4));
    if (!ok) r[s] = zero8();
  }
  if (KREM) {
    const bool low = (lane >> 4) < 2;
    r[KSTEPS] = *reinterpret_cast<const bf16x8*>(row + 32 * KSTEPS + 8 * ((lane >> 4) & 1));
    if (!ok || !low) r[KSTEPS] = zero8();
  }
}

struct Geometry {
  const uint16_t* k_pages;   // [pages, nkv, P, D]
  const uint16_t* v_pages;   // [pages, nkv, D, P]
  const int* bt;             // this request's block table row
  int nkv, g, page_shift, kv_len;
  float scale;
};

__device__ __forceinline__ s16x4 pack_bf16x4(float a, float b, float c, float d) {
  s16x4 r;
  r[0] = (short)float_to_bf16_bits(a);
  r[1] = (short)float_to_bf16_bits(b);
  r[2] = (short)float_to_bf16_bits(c);
  r[3] = (short)float_to_bf16_bits(d);
  return r;
}

// Loads the query rows of NB blocks of 16 columns.  Column c of block nb is token (first_col + 16 nb + c) / gpad
// of the entry, head (...) % gpad of the group; columns without a query hold zeros.
template <int NB>
__device__ __forceinline__ void load_queries(QRegs (&q)[NB], const uint16_t* q_base, int64_t q_row_stride, int first_col,
                                             int gpad, int G, int q_tokens, int head0) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int col = first_col + 16 * nb + (lane & 15);
    const int tok = col / gpad, hh = col % gpad;
    const bool ok = hh < G && tok < q_tokens;
    const uint16_t* row = q_base + (int64_t)(ok ? tok : 0) * q_row_stride + (int64_t)(head0 + (ok ? hh : 0)) * D;
    load_row(q[nb].full, row, ok);
  }
}

// Running softmax state of NB column blocks.
template <int NB>
struct State {
  float m[NB];        // running maximum of the column (same in the 4 lanes that share it)
  float l[NB];        // this lane's share of the running sum
  f32x4 o[NB][DBLK];  // O^T accumulators: dims 16 blk + 4 (lane / 16) + i of column lane % 16
};

// The cache operands of one tile of 16 keys in the lane's MFMA slots.
struct TileRegs {
  bf16x8 ka[QSTEPS];
  s16x4 va[DBLK];
};

// Page ids of the tile that starts at key j0 (addresses clamped to the request's last key: masked keys read
// valid memory of the request).
__device__ __forceinline__ void tile_pages(const Geometry& geo, int j0, int& kk, int& vk, int& kpage, int& vpage) {
  const int lane = threadIdx.x & 63;
  const int last = geo.kv_len - 1;
  kk = j0 + (lane & 15);
  kk = kk > last ? last : kk;
  vk = j0 + 4 * (lane >> 4);
  vk = vk > last ? (last & ~3) : vk;
  kpage = geo.bt[kk >> geo.page_shift];
  vpage = geo.bt[vk >> geo.page_shift];
}

__device__ __forceinline__ void tile_load(TileRegs& t, const Geometry& geo, int kk, int vk, int kpage, int vpage) {
  const int lane = threadIdx.x & 63;
  const int P = 1 << geo.page_shift;
  const uint16_t* krow = geo.k_pages + (((int64_t)kpage * geo.nkv + geo.g) * P + (kk & (P - 1))) * D;
  load_row(t.ka, krow, true);
  const uint16_t* vbase = geo.v_pages + (((int64_t)vpage * geo.nkv + geo.g) * D + (lane & 15)) * P + (vk & (P - 1));
#pragma unroll
  for (int blk = 0; blk < DBLK; ++blk) t.va[blk] = *reinterpret_cast<const s16x4*>(vbase + (int64_t)16 * blk * P);
}

// Scores, running softmax and the value product of one tile whose operands are in `t`.
template <int NB>
__device__ __forceinline__ void tile_compute(State<NB>& st, const QRegs (&q)[NB], const TileRegs& t, float scale, int j0,
                                             const int (&pos_lo)[NB], const int (&pos_hi)[NB]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < QSTEPS; ++k) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(t.ka[k], q[nb].full[k], s, 0, 0, 0);
    // lane holds S^T[key j0 + 4 (lane / 16) + i][column lane % 16]
    const int kbase = j0 + 4 * (lane >> 4);
    float sv[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int key = kbase + i;
      const bool ok = key <= pos_hi[nb] && key >= pos_lo[nb];
      sv[i] = ok ? s[i] * scale : -INFINITY;
      tmax = fmaxf(tmax, sv[i]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(st.m[nb], tmax);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;   // a column that has seen no key yet
    const float alpha = expf(st.m[nb] - m_use);               // exp(-inf) = 0 on the first visible tile
    float p[4];
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = expf(sv[i] - m_use);                             // exp(-inf) = 0 for masked keys
      psum += p[i];
    }
    st.l[nb] = st.l[nb] * alpha + psum;
    st.m[nb] = m_new;
    const s16x4 pb = pack_bf16x4(p[0], p[1], p[2], p[3]);
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk) {
      f32x4 o = st.o[nb][blk];
      o[0] *= alpha;
      o[1] *= alpha;
      o[2] *= alpha;
      o[3] *= alpha;
      st.o[nb][blk] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(t.va[blk], pb, o, 0, 0, 0);
    }
  }
}

// One pass over the tiles of 16 keys that start at key_begin, key_begin + stride, ... below key_end
// (key_begin a multiple of 16, stride a multiple of 16).
// pos_hi[nb] / pos_lo[nb]: the last and first key the lane's column of block nb may see (pos_hi < 0: none).
// (Running the loads a tile ahead of the arithmetic by hand was measured and gained nothing: the waves of a
// compute unit already overlap one another's loads.)
template <int NB>
__device__ __forceinline__ void attend(State<NB>& st, const QRegs (&q)[NB], const Geometry& geo, int key_begin,
                                       int key_end, int stride, const int (&pos_lo)[NB], const int (&pos_hi)[NB]) {
  for (int j0 = key_begin; j0 < key_end; j0 += stride) {
    TileRegs t;
    int kk, vk, kpage, vpage;
    tile_pages(geo, j0, kk, vk, kpage, vpage);
    tile_load(t, geo, kk, vk, kpage, vpage);
    tile_compute<NB>(st, q, t, geo.scale, j0, pos_lo, pos_hi);
  }
}

template <int NB>
__device__ __forceinline__ void init_state(State<NB>& st) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    st.m[nb] = -INFINITY;
    st.l[nb] = 0.f;
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk) st.o[nb][blk] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
}

// ---------------------------------------------------------------- prefill: several new tokens per entry
// work[w] = {entry b, block index within the entry}; a block is 16 * NB columns = 16 * NB / gpad query tokens.
template <int NB>
__global__ __launch_bounds__(256) void prefill_kernel(
    const uint16_t* __restrict__ q, int64_t q_row_stride, uint16_t* __restrict__ out, int64_t out_row_stride,
    const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ work, int num_work, const int* __restrict__ cu_q,
    const int* __restrict__ kv_len, int nq, int nkv, int gpad, int page_shift, float scale, int window) {
  const int lane = threadIdx.x & 63;
  const int w = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (w >= num_work) return;
  const int b = work[2 * w], blk_idx = work[2 * w + 1];
  const int g = blockIdx.y;
  const int G = nq / nkv;
  const int q_begin = cu_q[b];
  const int q_len = cu_q[b + 1] - q_begin;
  const int kv = kv_len[b];
  const int tokens_per_block = 16 * NB / gpad;
  const int tok0 = blk_idx * tokens_per_block;          // first query token of this block within the entry
  const int q_tokens = min(tokens_per_block, q_len - tok0);
  const int pos0 = kv - q_len + tok0;                   // its position

  Geometry geo{k_pages, v_pages, block_table + (int64_t)b * table_width, nkv, g, page_shift, kv, scale};
  QRegs qr[NB];
  load_queries<NB>(qr, q + (int64_t)(q_begin + tok0) * q_row_stride, q_row_stride, 0, gpad, G, q_tokens, g * G);

  int pos_lo[NB], pos_hi[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int col = 16 * nb + (lane & 15);
    const int tok = col / gpad, hh = col % gpad;
    const bool ok = hh < G && tok < q_tokens;
    pos_hi[nb] = ok ? pos0 + tok : -1;
    pos_lo[nb] = (ok && window > 0 && pos0 + tok - window + 1 > 0) ? pos0 + tok - window + 1 : 0;
  }
  const int first_pos = pos0, last_pos = pos0 + q_tokens - 1;
  const int lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;

  State<NB> st;
  init_state<NB>(st);
  attend<NB>(st, qr, geo, lo & ~15, last_pos + 1, 16, pos_lo, pos_hi);

#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float l = st.l[nb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (pos_hi[nb] < 0) continue;
    const float inv = 1.f / l;
    const int col = 16 * nb + (lane & 15);
    const int tok = col / gpad, hh = col % gpad;
    uint16_t* o = out + (int64_t)(q_begin + tok0 + tok) * out_row_stride + (int64_t)(g * G + hh) * D + 4 * (lane >> 4);
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk) {
      const f32x4 v = st.o[nb][blk];
      *reinterpret_cast<s16x4*>(o + 16 * blk) = pack_bf16x4(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
    }
  }
}

// ---------------------------------------------------------------- decode: one new token per entry, keys split
// Grid (num_splits, nkv, entries), 4 waves per workgroup.  The tiles of a split go round-robin to the waves, which
// combine their running softmax states through LDS.  With one split the workgroup writes the output itself;
// with several it writes a partial (max, sum, unnormalised output) per head, and the merge kernel below
// combines the partials with the log-sum-exp rule.  (Merging inside this kernel, by the workgroup that
// finishes last, was measured: the device-wide fences it needs cost many times the second launch.)
// Partials: part_o [entries, nq, num_splits, D], part_ml [entries, nq, num_splits, 2].
// (2 waves for the largest head sizes, whose states would not fit 64 KB of LDS fourfold)
constexpr int DECODE_WAVES = D > 128 ? 2 : 4;

__global__ __launch_bounds__(64 * DECODE_WAVES) void decode_kernel(
    const uint16_t* __restrict__ q, int64_t q_row_stride, uint16_t* __restrict__ out, int64_t out_row_stride,
    const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ cu_q, const int* __restrict__ kv_len, int first_entry,
    float* __restrict__ part_o, float* __restrict__ part_ml, int nq, int nkv, int page_shift, float scale, int window) {
  __shared__ float lds_o[DECODE_WAVES][DBLK][64][4];
  __shared__ float lds_m[DECODE_WAVES][16];
  __shared__ float lds_l[DECODE_WAVES][16];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int split = blockIdx.x, num_splits = gridDim.x;
  const int g = blockIdx.y;
  const int e = blockIdx.z;             // entry index among the decode entries
  const int b = first_entry + e;
  const int G = nq / nkv;
  const int kv = kv_len[b];
  const int pos = kv - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  // this split's keys: tiles of 16 from the first visible tile, evenly over the splits
  const int tile_lo = lo >> 4, tile_hi = (pos >> 4) + 1;
  const int tiles_per_split = (tile_hi - tile_lo + num_splits - 1) / num_splits;
  const int t0 = tile_lo + split * tiles_per_split;
  const int t1 = min(tile_hi, t0 + tiles_per_split);

  State<1> st;
  init_state<1>(st);
  const bool col_ok = (lane & 15) < G;
  {
    Geometry geo{k_pages, v_pages, block_table + (int64_t)b * table_width, nkv, g, page_shift, kv, scale};
    QRegs qr[1];
    load_queries<1>(qr, q + (int64_t)cu_q[b] * q_row_stride, q_row_stride, 0, 16, G, 1, g * G);
    const int pos_lo[1] = {lo};
    const int pos_hi[1] = {col_ok ? pos : -1};
    attend<1>(st, qr, geo, (t0 + wave) << 4, t1 << 4, 16 * DECODE_WAVES, pos_lo, pos_hi);
  }
  // ---- combine the waves: every wave leaves its state in LDS
  float l = st.l[0];
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
#pragma unroll
  for (int blk = 0; blk < DBLK; ++blk) *reinterpret_cast<f32x4*>(&lds_o[wave][blk][lane][0]) = st.o[0][blk];
  if (lane < 16) {
    lds_m[wave][lane] = st.m[0];
    lds_l[wave][lane] = l;
  }
  __syncthreads();
  // thread -> (block of dims, lane slot): column c = slot % 16, dims 16 blk + 4 (slot / 16) + i
  for (int idx = threadIdx.x; idx < DBLK * 64; idx += blockDim.x) {
    const int blk = idx >> 6, slot = idx & 63;
    const int c = slot & 15;
    if (c >= G) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < DECODE_WAVES; ++w) M = fmaxf(M, lds_m[w][c]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < DECODE_WAVES; ++w) {
      const float mw = lds_m[w][c];
      const float wt = (mw == -INFINITY) ? 0.f : expf(mw - M);
      const f32x4 v = *reinterpret_cast<const f32x4*>(&lds_o[w][blk][slot][0]);
      acc[0] += wt * v[0];
      acc[1] += wt * v[1];
      acc[2] += wt * v[2];
      acc[3] += wt * v[3];
      L += wt * lds_l[w][c];
    }
    const int head = g * G + c;
    const int dim = 16 * blk + 4 * (slot >> 4);
    if (num_splits == 1) {
      const float inv = 1.f / L;
      uint16_t* o = out + (int64_t)cu_q[b] * out_row_stride + (int64_t)head * D + dim;
      *reinterpret_cast<s16x4*>(o) = pack_bf16x4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
    } else {
      const int64_t ps = ((int64_t)e * nq + head) * num_splits + split;
      *reinterpret_cast<f32x4*>(part_o + ps * D + dim) = acc;
      if (blk == 0 && (slot >> 4) == 0) {
        part_ml[ps * 2] = M;
        part_ml[ps * 2 + 1] = L;
      }
    }
  }
}

// out[token of entry e][head] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s
// One wave per (entry, head).  The lanes first share out the splits (maximum, weights, sum), then the dims;
// the loads of a phase do not depend on one another, so they are all in flight together.
__global__ __launch_bounds__(64) void decode_merge_kernel(const float* __restrict__ part_o,
                                                          const float* __restrict__ part_ml,
                                                          uint16_t* __restrict__ out, int64_t out_row_stride,
                                                          const int* __restrict__ cu_q, int first_entry, int nq,
                                                          int num_splits) {
  const int lane = threadIdx.x;
  const int e = blockIdx.x / nq, head = blockIdx.x % nq;
  const int64_t base = ((int64_t)e * nq + head) * num_splits;
  constexpr int MAXR = 16;
  float mv[MAXR], lv[MAXR];
  float M = -INFINITY;
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    const int s = lane + 64 * r;
    const bool ok = s < num_splits;
    const float2 ml = ok ? *reinterpret_cast<const float2*>(part_ml + (base + s) * 2) : float2{-INFINITY, 0.f};
    mv[r] = ml.x;
    lv[r] = ml.y;
    M = fmaxf(M, ml.x);
    if (64 * (r + 1) >= num_splits) break;
  }
  M = wave_max(M);
  float L = 0.f;
#pragma unroll
  for (int r = 0; r < MAXR; ++r) {
    mv[r] = (mv[r] == -INFINITY) ? 0.f : expf(mv[r] - M);
    L += mv[r] * lv[r];
    if (64 * (r + 1) >= num_splits) break;
  }
  L = wave_sum(L);
  const float inv = 1.f / L;
  uint16_t* o = out + (int64_t)cu_q[first_entry + e] * out_row_stride + (int64_t)head * D;
#pragma unroll
  for (int round = 0; round < (D + 255) / 256; ++round) {
    const int dd = 256 * round + 4 * lane;
    const bool live = dd < D;
    const int d0 = live ? dd : 0;
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < MAXR; ++r) {
      const int n = min(64, num_splits - 64 * r);
#pragma unroll 8
      for (int j = 0; j < n; ++j) {
        const float w = __shfl(mv[r], j, 64);
        const f32x4 v = *reinterpret_cast<const f32x4*>(part_o + (base + 64 * r + j) * D + d0);
        acc[0] += w * v[0];
        acc[1] += w * v[1];
        acc[2] += w * v[2];
        acc[3] += w * v[3];
      }
      if (64 * (r + 1) >= num_splits) break;
    }
    if (live) *reinterpret_cast<s16x4*>(o + d0) = pack_bf16x4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
  }
}

// ---------------------------------------------------------------- entry points
static int check_common(const char* what, int nq, int nkv, int page_size, int64_t q_row_stride, int64_t out_row_stride,
                        int table_width) {
  MI_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "%s: %d query heads are no multiple of %d kv heads", what, nq, nkv);
  MI_REQUIRE(nq / nkv <= 16, "%s: %d query heads per kv head; this kernel takes at most 16", what, nq / nkv);
  MI_REQUIRE(page_size >= 4 && (page_size & (page_size - 1)) == 0, "%s: page size %d is not a power of two >= 4", what,
             page_size);
  MI_REQUIRE(q_row_stride >= (int64_t)nq * D && q_row_stride % 8 == 0, "%s: query row stride %lld", what,
             (long long)q_row_stride);
  MI_REQUIRE(out_row_stride >= (int64_t)nq * D && out_row_stride % 4 == 0, "%s: output row stride %lld", what,
             (long long)out_row_stride);
  MI_REQUIRE(table_width > 0, "%s: empty block table", what);
  return 0;
}

static int log2_of(int v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

MI_EXPORT int mi_attn_head_dim() { return D; }

// Columns per block and query tokens per block for `nq / nkv` heads per group.
MI_EXPORT int mi_attn_prefill_tokens_per_block(int nq, int nkv) {
  const int G = nq / nkv;
  int gpad = 1;
  while (gpad < G) gpad <<= 1;
  return gpad > 16 ? 0 : 32 / gpad;
}

MI_EXPORT int mi_attn_prefill(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride, const void* k_pages,
                              const void* v_pages, const int* block_table, int table_width, const int* work,
                              int num_work, const int* cu_q, const int* kv_len, int nq, int nkv, int page_size,
                              float scale, int window, hipStream_t stream) {
  if (check_common("attn_prefill", nq, nkv, page_size, q_row_stride, out_row_stride, table_width)) return 1;
  MI_REQUIRE(num_work >= 0 && window >= 0, "attn_prefill: bad work count or window");
  if (num_work == 0) return 0;
  const int G = nq / nkv;
  int gpad = 1;
  while (gpad < G) gpad <<= 1;
  dim3 grid((num_work + 3) / 4, nkv);
  prefill_kernel<2><<<grid, 256, 0, stream>>>((const uint16_t*)q, q_row_stride, (uint16_t*)out, out_row_stride,
                                              (const uint16_t*)k_pages, (const uint16_t*)v_pages, block_table,
                                              table_width, work, num_work, cu_q, kv_len, nq, nkv, gpad,
                                              log2_of(page_size), scale, window);
  MI_CHECK_LAUNCH("attn_prefill");
  return 0;
}

// Entries first_entry .. first_entry + num_entries - 1 must each bring exactly one token.
// part_o: float [num_entries * nq * num_splits * D]; part_ml: float [num_entries * nq * num_splits * 2].
MI_EXPORT int mi_attn_decode(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride, const void* k_pages,
                             const void* v_pages, const int* block_table, int table_width, const int* cu_q,
                             const int* kv_len, int first_entry, int num_entries, int num_splits, float* part_o,
                             float* part_ml, int nq, int nkv, int page_size, float scale, int window,
                             hipStream_t stream) {
  if (check_common("attn_decode", nq, nkv, page_size, q_row_stride, out_row_stride, table_width)) return 1;
  MI_REQUIRE(num_entries >= 0 && first_entry >= 0 && window >= 0, "attn_decode: bad entry range or window");
  MI_REQUIRE(num_splits >= 1 && num_splits <= 1024, "attn_decode: %d splits", num_splits);
  MI_REQUIRE(num_entries <= 65535 && nkv <= 65535, "attn_decode: grid too large");
  MI_REQUIRE(num_splits == 1 || (part_o && part_ml), "attn_decode: no partial buffers");
  if (num_entries == 0) return 0;
  dim3 grid(num_splits, nkv, num_entries);
  decode_kernel<<<grid, 64 * DECODE_WAVES, 0, stream>>>(
      (const uint16_t*)q, q_row_stride, (uint16_t*)out, out_row_stride, (const uint16_t*)k_pages,
      (const uint16_t*)v_pages, block_table, table_width, cu_q, kv_len, first_entry, part_o, part_ml, nq, nkv,
      log2_of(page_size), scale, window);
  MI_CHECK_LAUNCH("attn_decode");
  if (num_splits > 1) {
    decode_merge_kernel<<<num_entries * nq, 64, 0, stream>>>(part_o, part_ml, (uint16_t*)out, out_row_stride, cu_q,
                                                             first_entry, nq, num_splits);
    MI_CHECK_LAUNCH("attn_decode merge");
  }
  return 0;
}
