// bfloat16 attention over the paged cache on the matrix cores (MFMA) of gfx950, for one head size
// (compile with -DHEAD_DIM=<multiple of 16, at most 256>).
//
// Same function as attention.hip (bottom-right aligned causal mask, optional window, grouped heads:
// miniinfer/layers/attention.py:112-191), in two launches:
//   prefill: entries with several new tokens; a workgroup of 4 waves takes 4 blocks of query columns of one
//            entry and kv head and shares each tile of keys and values through LDS;
//   decode:  entries with one new token; the keys of a request are split over workgroups (flash-decoding),
//            which write (max, sum, unnormalised output) partials that a merge kernel combines with the
//            log-sum-exp rule.
//
// Layout of the products, chosen so that every operand comes straight from memory or from the previous
// product's accumulators:
//   S^T[key, col] = K[key, :] . Q[col, :]      A = K rows (16 B per lane from a key's row), B = Q rows
//   O^T[dim, col] = V^T[dim, :] . P^T[:, col]  A = V^T rows (value pages are stored [dim][key in page]),
//                                              B = P, which is exactly where S^T's accumulators sit
// A "column" is a (query token, query head of the kv group) pair; 16 columns form an MFMA block.  All
// softmax statistics of a column live in the lanes with lane % 16 == column.  Scores, softmax and
// accumulation are 32-bit; P is rounded to bfloat16 for the second product.
//
// The running softmax is updated once per macro tile of MT * 16 keys (one maximum, one rescale of the output
// accumulators, and that only when some column's maximum moved), in base 2: scores are scaled by
// scale * log2(e), so a probability is one v_exp_f32.
#include "common.h"
#include "attention_mfma.h"

#include <mutex>

#ifndef HEAD_DIM
#error "compile with -DHEAD_DIM=<head size>"
#endif
static_assert(HEAD_DIM % 16 == 0 && HEAD_DIM >= 16 && HEAD_DIM <= 256, "head size must be a multiple of 16 up to 256");

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // (arrays of HIP's uint4 class end up in scratch memory)
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int D = HEAD_DIM;

// Register budgets.  Up to head size 128 the decode kernel is held to the registers that let two waves share a
// SIMD (the compiler would otherwise take a few more and lose a wave to them), and the prefill kernel exists a
// second time, held to three waves per SIMD at the price of a few spilled registers: that pays when there are
// more than two workgroups for every compute unit, and costs when there are not.
#if HEAD_DIM <= 128
#define DECODE_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2)))
#define PREFILL_DENSE_OCCUPANCY __attribute__((amdgpu_waves_per_eu(3)))
#define PREFILL_WIDE 1          // a third prefill instance: two blocks of query columns per wave, two waves per SIMD
#else
#define DECODE_OCCUPANCY
#define PREFILL_DENSE_OCCUPANCY
#define PREFILL_WIDE 0          // (its accumulators alone would fill the registers of head sizes above 128)
#endif
constexpr int KSTEPS = D / 32;          // 16x16x32 products over the head dim
constexpr bool KREM = (D % 32) != 0;    // plus one more, half of it zeros
constexpr int QSTEPS = KSTEPS + (KREM ? 1 : 0);
constexpr int DBLK = D / 16;            // 16-row blocks of O^T
constexpr int MT = D > 128 ? 2 : 4;     // tiles of 16 keys per macro tile
constexpr int MKEYS = 16 * MT;          // keys per macro tile
static_assert(MT % 2 == 0, "the second product takes the tiles in pairs");

// The last 16 dims of a head size that is no multiple of 32 go through the same 16x16x32 product with the
// upper half of the contraction zeroed: lanes 0..31 hold 8 dims each, lanes 32..63 hold zeros.  (Finishing
// the score with a 16x16x16 product on the accumulator of the 16x16x32 ones gave wrong sums on gfx950 with
// hipcc 7.2 whenever a wave ran more than one tile; one opcode per accumulator chain does not.)
struct QRegs {
  bf16x8 full[QSTEPS];
};

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

// operand registers of one row (a key's or a query's D elements) in the lane's MFMA slots
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

// the same for a row that is read once and should not push anything else out of the caches (a decode step's keys)
__device__ __forceinline__ void load_row_stream(bf16x8 (&r)[QSTEPS], const uint16_t* row) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int s = 0; s < KSTEPS; ++s)
    r[s] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(row + 32 * s + 8 * (lane >> 4)));
  if (KREM) {
    const bool low = (lane >> 4) < 2;
    r[KSTEPS] = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(row + 32 * KSTEPS + 8 * ((lane >> 4) & 1)));
    if (!low) r[KSTEPS] = zero8();
  }
}

// two floats -> two bfloat16 in one register (v_cvt_pk_bf16_f32, round to nearest even)
__device__ __forceinline__ uint32_t pack_bf16x2(float a, float b) {
  const f32x2 v = {a, b};
  const bf16x2 r = __builtin_convertvector(v, bf16x2);
  return *reinterpret_cast<const uint32_t*>(&r);
}

__device__ __forceinline__ s16x4 pack_bf16x4(float a, float b, float c, float d) {
  union {
    uint32_t u[2];
    s16x4 v;
  } r;
  r.u[0] = pack_bf16x2(a, b);
  r.u[1] = pack_bf16x2(c, d);
  return r.v;
}

// Loads the query rows of NB blocks of 16 columns.  Column c of block nb is token (16 nb + c) / gpad of the
// `q_tokens` tokens that start at q_base, head (16 nb + c) % gpad of the group; columns without a query hold zeros.
template <int NB>
__device__ __forceinline__ void load_queries(QRegs (&q)[NB], const uint16_t* q_base, int64_t q_row_stride, int gpad,
                                             int G, int q_tokens, int head0) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int col = 16 * nb + (lane & 15);
    const int tok = col / gpad, hh = col % gpad;
    const bool ok = hh < G && tok < q_tokens;
    const uint16_t* row = q_base + (int64_t)(ok ? tok : 0) * q_row_stride + (int64_t)(head0 + (ok ? hh : 0)) * D;
    load_row(q[nb].full, row, ok);
  }
}

// Running softmax state of NB column blocks (maxima in base-2 units of the scaled scores).
template <int NB>
struct State {
  float m[NB];        // running maximum of the column (same in the 4 lanes that share it)
  float l[NB];        // this lane's share of the running sum
  f32x4 o[NB][DBLK];  // O^T accumulators: dims 16 blk + 4 (lane / 16) + i of column lane % 16
};

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

// S^T of one tile of 16 keys (operands `ka`) against the NB query blocks.
template <int NB>
__device__ __forceinline__ void tile_scores(f32x4 (&s)[NB], const bf16x8 (&ka)[QSTEPS], const QRegs (&q)[NB]) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int k = 0; k < QSTEPS; ++k) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[k], q[nb].full[k], acc, 0, 0, 0);
    s[nb] = acc;
  }
}

// The running softmax over the macro tile that starts at key j0: masks the scores in s[t][nb] (lane: key
// j0 + 16 t + 4 (lane / 16) + i, column lane % 16), moves the maxima, rescales sums and accumulators, and leaves
// the probabilities, rounded to bfloat16, in p[t][nb].  c = scale * log2(e) > 0; the scale is folded into the
// exponent's multiply-add, so a probability costs a max, an fma, an exp2 and an add.
// pos_hi[nb] / pos_lo[nb]: the last and first key the lane's column of block nb may see (pos_hi < 0: none).
// Most macro tiles lie wholly inside every column's range; those skip the masking (the test is per wave).
template <int NB>
__device__ __forceinline__ void softmax_update(State<NB>& st, f32x4 (&s)[MT][NB], s16x4 (&p)[MT][NB], float c, int j0,
                                               const int (&pos_lo)[NB], const int (&pos_hi)[NB]) {
  const int lane = threadIdx.x & 63;
  const int kbase = j0 + 4 * (lane >> 4);
  bool inside = true;                    // columns without a query do not matter: their results are dropped
#pragma unroll
  for (int nb = 0; nb < NB; ++nb)
    inside = inside && (pos_hi[nb] < 0 || (j0 + MKEYS - 1 <= pos_hi[nb] && j0 >= pos_lo[nb]));
  const bool full = __all(inside);
  float alpha[NB];
  bool moved = false;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float tmax = -INFINITY;
    if (full) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) tmax = fmaxf(tmax, s[t][nb][i]);
    } else {
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = kbase + 16 * t + i;
          const bool ok = key <= pos_hi[nb] && key >= pos_lo[nb];
          const float v = ok ? s[t][nb][i] : -INFINITY;
          s[t][nb][i] = v;
          tmax = fmaxf(tmax, v);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(st.m[nb], tmax * c);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;    // a column that has seen no key yet
    alpha[nb] = __builtin_amdgcn_exp2f(st.m[nb] - m_use);      // 2^-inf = 0 on the first visible tile
    moved = moved || (m_new != st.m[nb]);
    float psum = 0.f;
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float e[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        e[i] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[t][nb][i], c, -m_use));    // 0 for masked keys
        psum += e[i];
      }
      p[t][nb] = pack_bf16x4(e[0], e[1], e[2], e[3]);
    }
    st.l[nb] = st.l[nb] * alpha[nb] + psum;
    st.m[nb] = m_new;
  }
  if (__any(moved)) {     // the same for every lane of the wave
#pragma unroll
    for (int nb = 0; nb < NB; ++nb)
#pragma unroll
      for (int blk = 0; blk < DBLK; ++blk) {
        st.o[nb][blk][0] *= alpha[nb];
        st.o[nb][blk][1] *= alpha[nb];
        st.o[nb][blk][2] *= alpha[nb];
        st.o[nb][blk][3] *= alpha[nb];
      }
  }
}

// O^T += V^T P^T for two tiles of 16 keys at once (operands va0 / p0 of one tile, va1 / p1 of the other), as one
// 16x16x32 product: the order of the contraction index is free as long as both operands agree, so slot 8 q + e of
// lane group q is key 4 q + e of the first tile for e < 4 and key 4 q + e - 4 of the second for e >= 4, which is
// where the values' 8-byte reads and the first product's accumulators already are.
__device__ __forceinline__ bf16x8 join8(const s16x4 lo, const s16x4 hi) {
  union {
    s16x4 h[2];
    bf16x8 v;
  } u;
  u.h[0] = lo;
  u.h[1] = hi;
  return u.v;
}

template <int NB>
__device__ __forceinline__ void tile_values(State<NB>& st, const s16x4 (&va0)[DBLK], const s16x4 (&va1)[DBLK],
                                            const s16x4 (&p0)[NB], const s16x4 (&p1)[NB]) {
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const bf16x8 pb = join8(p0[nb], p1[nb]);
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk)
      st.o[nb][blk] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(join8(va0[blk], va1[blk]), pb, st.o[nb][blk], 0, 0, 0);
  }
}

// Normalises and stores the columns of a wave: token col / gpad of the rows that start at out_base.
template <int NB>
__device__ __forceinline__ void store_output(const State<NB>& st, uint16_t* out_base, int64_t out_row_stride, int gpad,
                                             int head0, const int (&pos_hi)[NB]) {
  const int lane = threadIdx.x & 63;
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    float l = st.l[nb];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (pos_hi[nb] < 0) continue;
    const float inv = 1.f / l;
    const int col = 16 * nb + (lane & 15);
    const int tok = col / gpad, hh = col % gpad;
    uint16_t* o = out_base + (int64_t)tok * out_row_stride + (int64_t)(head0 + hh) * D + 4 * (lane >> 4);
#pragma unroll
    for (int blk = 0; blk < DBLK; ++blk) {
      const f32x4 v = st.o[nb][blk];
      *reinterpret_cast<s16x4*>(o + 16 * blk) = pack_bf16x4(v[0] * inv, v[1] * inv, v[2] * inv, v[3] * inv);
    }
  }
}

// ---------------------------------------------------------------- prefill: several new tokens per entry
// A workgroup of 4 waves takes 4 consecutive query blocks of one entry and one kv head.  All four need the same
// keys and values, so each macro tile is read from global memory once per workgroup, by all 256 threads
// together, into LDS (the next tile's loads are in flight in registers while the current one is multiplied), and
// every wave takes its MFMA operands from there.  Rows are padded so that the 16 lanes of an operand read hit
// different banks.  work[w] = {entry, block of 4 * (16 NB / gpad) query tokens}.  Pages hold 8 tokens or more.
#ifndef PREFILL_NB
#define PREFILL_NB 1
#endif
// Elements per key row in LDS.  An operand read takes 16 bytes per lane from 16 rows (lanes l and l + 16 read
// neighbouring pieces of a row); the LDS serves lanes l .. l + 3 and l + 16 .. l + 19 together, so these 4 rows x 2
// pieces must fall into different banks: a row stride of 8 (mod 16) banks of 4 bytes, D + 16 elements for head
// sizes that are multiples of 32 and D itself for the others.  (With D + 8 a third of the kernel's LDS cycles
// were bank conflicts of these reads: SQ_LDS_BANK_CONFLICT 2.0e8 against 0.7e8 for 16,384 tokens.)
constexpr int LDS_KSTR = (D % 32 == 0) ? D + 16 : D;
constexpr int LDS_VSTR = MKEYS + 4;              // elements per dim row of the transposed values in LDS: rows 2 banks
                                                 // apart, so the 16 rows x 8 bytes of an operand read hit 32 banks
constexpr int LDS_KCHUNKS = MKEYS * (D / 8);     // 16-byte chunks of a key tile
constexpr int LDS_VCHUNKS = D * (MKEYS / 8);     // 16-byte chunks of a value tile
constexpr int LDS_KITER = (LDS_KCHUNKS + 255) / 256;
constexpr int LDS_VITER = (LDS_VCHUNKS + 255) / 256;

// KG = 1: as described.  KG = 2: the workgroup has 8 waves and walks two macro tiles per step, staged side by side;
// waves 0-3 take the first of each pair, waves 4-7 the second, for the same 4 query blocks, and at the end wave
// w + 4 hands its running softmax state to wave w through LDS.  That halves the number of dependent steps of the
// workgroup with the most keys, which is what a short prompt's launch waits for.
template <int NB, int KG>
__device__ __forceinline__ void prefill_body(
    const uint16_t* __restrict__ q, int64_t q_row_stride, uint16_t* __restrict__ out, int64_t out_row_stride,
    const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ work, const int* __restrict__ cu_q, const int* __restrict__ kv_len, int nq,
    int nkv, int gpad, int page_shift, float scale, int window) {
  constexpr int KS_TILE = MKEYS * LDS_KSTR, VS_TILE = D * LDS_VSTR;
  __shared__ __attribute__((aligned(16))) uint16_t tiles[KG * (KS_TILE + VS_TILE)];   // keys, then values
  uint16_t* Ks_all = tiles;
  uint16_t* Vs_all = tiles + KG * KS_TILE;
  static_assert((KG * KS_TILE) % 8 == 0, "the value tiles start on a 16-byte boundary");
  static_assert(KG == 1 || (size_t)(KS_TILE + VS_TILE) * KG * 2 >= (size_t)4 * NB * (DBLK * 64 * 4 + 128) * 4,
                "the tiles' LDS must hold four waves' states at the end");
  const int lane = threadIdx.x & 63;
  const int kgroup = (threadIdx.x >> 6) >> 2;            // which macro tile of a step this wave multiplies
  const int wave = (threadIdx.x >> 6) & 3;               // its query block within the workgroup
  const int tid = threadIdx.x & 255;                     // the thread's place among those that stage one macro tile
  // and which macro tile of a step they stage (the same for a whole wave: said so, for the scalar page lookups)
  const int stage = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);
  uint16_t* Ks = Ks_all + kgroup * KS_TILE;
  uint16_t* Vs = Vs_all + kgroup * VS_TILE;
  uint16_t* Ks_stage = Ks_all + stage * KS_TILE;
  uint16_t* Vs_stage = Vs_all + stage * VS_TILE;
  // The kv head is the fastest grid index: workgroups go round the 8 XCDs by their linear index, so with 8 kv
  // heads (or a divisor or multiple of 8) all the workgroups that read one head's keys and values share an L2.
  const int b = work[2 * blockIdx.y], sb = work[2 * blockIdx.y + 1];
  const int g = blockIdx.x;
  const int G = nq / nkv;
  const int P = 1 << page_shift;
  const int q_begin = cu_q[b];
  const int q_len = cu_q[b + 1] - q_begin;
  const int kv = kv_len[b];
  const int last = kv - 1;
  const int tokens_per_wave = 16 * NB / gpad;
  const int wg_tok0 = sb * 4 * tokens_per_wave;                    // first query token of the workgroup
  const int wg_tokens = min(4 * tokens_per_wave, q_len - wg_tok0);
  const int tok0 = wg_tok0 + wave * tokens_per_wave;               // of this wave
  const int q_tokens = max(0, min(tokens_per_wave, q_len - tok0));
  const int pos0 = kv - q_len + tok0;
  const int* bt = block_table + (int64_t)b * table_width;

  QRegs qr[NB];
  load_queries<NB>(qr, q + (int64_t)(q_begin + (q_tokens > 0 ? tok0 : wg_tok0)) * q_row_stride, q_row_stride, gpad, G,
                   q_tokens, g * G);
  int pos_lo[NB], pos_hi[NB];
#pragma unroll
  for (int nb = 0; nb < NB; ++nb) {
    const int col = 16 * nb + (lane & 15);
    const int tok = col / gpad, hh = col % gpad;
    const bool ok = hh < G && tok < q_tokens;
    pos_hi[nb] = ok ? pos0 + tok : -1;
    pos_lo[nb] = (ok && window > 0 && pos0 + tok - window + 1 > 0) ? pos0 + tok - window + 1 : 0;
  }
  // keys the workgroup walks, and the part of them this wave's queries can see
  const int wg_first = kv - q_len + wg_tok0, wg_last = wg_first + wg_tokens - 1;
  const int wg_lo = ((window > 0 && wg_first - window + 1 > 0) ? wg_first - window + 1 : 0) / MKEYS * MKEYS;
  const int wg_hi = wg_last + 1;
  const int w_lo = (q_tokens > 0 && window > 0 && pos0 - window + 1 > 0) ? pos0 - window + 1 : 0;
  const int w_hi = q_tokens > 0 ? pos0 + q_tokens : 0;
  const float c = scale * 1.44269504088896340736f;

  State<NB> st;
  init_state<NB>(st);

  // This thread's chunks of a macro tile: page numbers from the block table (PREFILL_PAGES), global -> registers
  // (PREFILL_FETCH), registers -> LDS (PREFILL_STASH).  The page numbers are asked for one tile earlier than the
  // keys and values that need them, so that no step of the loop waits for two dependent loads in a row.
  // Everything about a chunk that does not change from tile to tile is worked out once: which key of the tile
  // and which 16 bytes of it (keys), which dim and which run of 8 keys (values; chunk -> (page of the tile, dim,
  // run) so that consecutive threads read consecutive memory of a page), and where it goes in LDS.
  const int kpp = P < MKEYS ? P : MKEYS;   // keys of a macro tile that lie in one page
  const int cpp = kpp / 8;                 // 16-byte chunks per (page, dim)
  u32x4 pk[LDS_KITER], pv[LDS_VITER];
  int kpage[LDS_KITER], vpage[LDS_VITER];
  int k_key[LDS_KITER], k_col[LDS_KITER], k_lds[LDS_KITER];    // key in the tile, first element, LDS element offset
  int v_key[LDS_VITER], v_dim[LDS_VITER], v_lds[LDS_VITER];    // first key of the run in the tile, dim, LDS offset
#pragma unroll
  for (int it = 0; it < LDS_KITER; ++it) {
    int ch = tid + 256 * it;
    k_lds[it] = ch < LDS_KCHUNKS ? (ch / (D / 8)) * LDS_KSTR + 8 * (ch % (D / 8)) : -1;
    ch = ch < LDS_KCHUNKS ? ch : LDS_KCHUNKS - 1;   // threads past the end load the last chunk again and drop it
    k_key[it] = ch / (D / 8);
    k_col[it] = 8 * (ch % (D / 8));
  }
#pragma unroll
  for (int it = 0; it < LDS_VITER; ++it) {
    int ch = tid + 256 * it;
    const bool live = ch < LDS_VCHUNKS;
    ch = live ? ch : LDS_VCHUNKS - 1;
    const int part = ch % cpp, dim = (ch / cpp) % D, page_i = ch / (cpp * D);
    v_key[it] = page_i * kpp + 8 * part;
    v_dim[it] = dim;
    v_lds[it] = live ? dim * LDS_VSTR + page_i * kpp + 8 * part : -1;
  }
  const uint16_t* kbase = k_pages + (int64_t)g * P * D;     // + page * page_stride + (slot in page) * D + element
  const uint16_t* vbase = v_pages + (int64_t)g * D * P;     // + page * page_stride + dim * P + slot in page
  const int page_stride = nkv * P * D;                      // elements; a page of one layer is far below 2^31
  // For head sizes that are multiples of 64 (pages hold 8 tokens or more) the 64 chunks of a wave lie in one page,
  // keys and values alike: the page number is then looked up once per wave with scalar instructions (from the
  // first lane's key), and the page's base address is scalar arithmetic instead of 64-bit vector arithmetic
  // (about a quarter of the vector instructions that fetching a macro tile took).
  constexpr bool PAGE_PER_WAVE = (D % 64) == 0;
#define PREFILL_PAGES(J0)                                                                                            \
  {                                                                                                                  \
    _Pragma("unroll") for (int it = 0; it < LDS_KITER; ++it) {                                                       \
      int key = min((J0) + k_key[it], last); /* masked keys read valid memory of the request */                     \
      if (PAGE_PER_WAVE) key = __builtin_amdgcn_readfirstlane(key);                                                  \
      kpage[it] = bt[key >> page_shift];                                                                             \
    }                                                                                                                \
    _Pragma("unroll") for (int it = 0; it < LDS_VITER; ++it) {                                                       \
      int key = (J0) + v_key[it];                                                                                    \
      key = key > last ? (last & ~7) : key; /* a run of 8 keys lies in one page */                                  \
      if (PAGE_PER_WAVE) key = __builtin_amdgcn_readfirstlane(key);                                                  \
      vpage[it] = bt[key >> page_shift];                                                                             \
    }                                                                                                                \
  }
#define PREFILL_FETCH(J0)                                                                                            \
  {                                                                                                                  \
    _Pragma("unroll") for (int it = 0; it < LDS_KITER; ++it) {                                                       \
      const int key = min((J0) + k_key[it], last);                                                                   \
      const uint16_t* page = kbase + (int64_t)kpage[it] * page_stride;                                               \
      pk[it] = *reinterpret_cast<const u32x4*>(page + ((key & (P - 1)) * D + k_col[it]));                            \
    }                                                                                                                \
    _Pragma("unroll") for (int it = 0; it < LDS_VITER; ++it) {                                                       \
      int key = (J0) + v_key[it];                                                                                    \
      key = key > last ? (last & ~7) : key;                                                                          \
      const uint16_t* page = vbase + (int64_t)vpage[it] * page_stride;                                               \
      pv[it] = *reinterpret_cast<const u32x4*>(page + (v_dim[it] * P + (key & (P - 1))));                            \
    }                                                                                                                \
  }
#define PREFILL_STASH()                                                                                              \
  {                                                                                                                  \
    _Pragma("unroll") for (int it = 0; it < LDS_KITER; ++it)                                                         \
      if (k_lds[it] >= 0) *reinterpret_cast<u32x4*>(Ks_stage + k_lds[it]) = pk[it];                                  \
    _Pragma("unroll") for (int it = 0; it < LDS_VITER; ++it)                                                         \
      if (v_lds[it] >= 0) { /* rows are 8-byte aligned only: two 64-bit writes */                                    \
        u32x2* dst = reinterpret_cast<u32x2*>(Vs_stage + v_lds[it]);                                                 \
        dst[0] = u32x2{pv[it][0], pv[it][1]};                                                                        \
        dst[1] = u32x2{pv[it][2], pv[it][3]};                                                                        \
      }                                                                                                              \
  }

  // a thread stages the macro tile `stage` of every step; a wave multiplies the macro tile `kgroup` of every step
  constexpr int STEP = MKEYS * KG;
  const int s_off = MKEYS * stage, c_off = MKEYS * kgroup;
  PREFILL_PAGES(wg_lo + s_off)
  PREFILL_FETCH(wg_lo + s_off)
  PREFILL_PAGES(wg_lo + STEP + s_off)
  for (int j0 = wg_lo; j0 < wg_hi; j0 += STEP) {
    __syncthreads();                    // every wave is done with the tiles that are in LDS
    PREFILL_STASH()
    __syncthreads();
    if (j0 + STEP < wg_hi) {
      PREFILL_FETCH(j0 + STEP + s_off)
      PREFILL_PAGES(j0 + 2 * STEP + s_off)
    }
    const int jt = j0 + c_off;          // this wave's macro tile
    if (jt >= w_hi || jt + MKEYS <= w_lo) continue;      // nothing this wave can see (same for all its lanes)
    f32x4 s[MT][NB];
    s16x4 p[MT][NB];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      bf16x8 ka[QSTEPS];
      load_row(ka, Ks + (16 * t + (lane & 15)) * LDS_KSTR, true);
      tile_scores<NB>(s[t], ka, qr);
    }
    softmax_update<NB>(st, s, p, c, jt, pos_lo, pos_hi);
#pragma unroll
    for (int t = 0; t < MT; t += 2) {
      s16x4 va[2][DBLK];
#pragma unroll
      for (int u = 0; u < 2; ++u)
#pragma unroll
        for (int blk = 0; blk < DBLK; ++blk)
          va[u][blk] = *reinterpret_cast<const s16x4*>(Vs + (16 * blk + (lane & 15)) * LDS_VSTR + 16 * (t + u) +
                                                       4 * (lane >> 4));
      tile_values<NB>(st, va[0], va[1], p[t], p[t + 1]);
    }
  }
#undef PREFILL_PAGES
#undef PREFILL_FETCH
#undef PREFILL_STASH
  if constexpr (KG == 2) {
    // wave w + 4 leaves its state where the tiles were; wave w folds it into its own (log-sum-exp rule, base 2)
    __syncthreads();
    float* hand = reinterpret_cast<float*>(Ks_all) + wave * NB * (DBLK * 256 + 128);
    if (kgroup == 1) {
#pragma unroll
      for (int nb = 0; nb < NB; ++nb) {
        float* h = hand + nb * (DBLK * 256 + 128);
#pragma unroll
        for (int blk = 0; blk < DBLK; ++blk) *reinterpret_cast<f32x4*>(h + (blk * 64 + lane) * 4) = st.o[nb][blk];
        h[DBLK * 256 + lane] = st.m[nb];
        h[DBLK * 256 + 64 + lane] = st.l[nb];
      }
    }
    __syncthreads();
    if (kgroup == 1) return;
#pragma unroll
    for (int nb = 0; nb < NB; ++nb) {
      const float* h = hand + nb * (DBLK * 256 + 128);
      const float m1 = h[DBLK * 256 + lane], l1 = h[DBLK * 256 + 64 + lane];
      const float m_new = fmaxf(st.m[nb], m1);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float a0 = __builtin_amdgcn_exp2f(st.m[nb] - m_use), a1 = __builtin_amdgcn_exp2f(m1 - m_use);
      st.m[nb] = m_new;
      st.l[nb] = st.l[nb] * a0 + l1 * a1;
#pragma unroll
      for (int blk = 0; blk < DBLK; ++blk) {
        const f32x4 o1 = *reinterpret_cast<const f32x4*>(h + (blk * 64 + lane) * 4);
        st.o[nb][blk] = st.o[nb][blk] * a0 + o1 * a1;
      }
    }
  }
  store_output<NB>(st, out + (int64_t)(q_begin + tok0) * out_row_stride, out_row_stride, gpad, g * G, pos_hi);
}

#define PREFILL_ARGS                                                                                                 \
  const uint16_t *__restrict__ q, int64_t q_row_stride, uint16_t *__restrict__ out, int64_t out_row_stride,          \
      const uint16_t *__restrict__ k_pages, const uint16_t *__restrict__ v_pages, const int *__restrict__ block_table, \
      int table_width, const int *__restrict__ work, const int *__restrict__ cu_q, const int *__restrict__ kv_len,   \
      int nq, int nkv, int gpad, int page_shift, float scale, int window
#define PREFILL_PASS                                                                                                 \
  q, q_row_stride, out, out_row_stride, k_pages, v_pages, block_table, table_width, work, cu_q, kv_len, nq, nkv,     \
      gpad, page_shift, scale, window

template <int NB>
__global__ __launch_bounds__(512) void prefill_kernel(PREFILL_ARGS) {      // few workgroups: 8 waves, two tiles a step
  prefill_body<NB, 2>(PREFILL_PASS);
}

template <int NB>
__global__ __launch_bounds__(256) PREFILL_DENSE_OCCUPANCY void prefill_dense_kernel(PREFILL_ARGS) {
  prefill_body<NB, 1>(PREFILL_PASS);
}

// Long prompts (many workgroups for every compute unit): every wave takes two blocks of 16 query columns, so a
// tile's operands, read from LDS once per wave, serve twice the products (what the instances above wait for is
// those LDS reads and the vector work of fetching a tile, the same per tile whatever a wave multiplies it with):
// 246 registers at head size 128, two waves per SIMD, no spills.  32,768 tokens: 789 against 665 TFLOP/s; 8,192:
// 672 against 619; for short prompts it has too few workgroups (2,048 tokens: 82 against 52 us).
#if PREFILL_WIDE
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void prefill_wide_kernel(PREFILL_ARGS) {
  prefill_body<2, 1>(PREFILL_PASS);
}
#endif
#undef PREFILL_ARGS
#undef PREFILL_PASS

// ---------------------------------------------------------------- decode: one new token per entry, keys split
// Grid (num_splits, nkv, entries), DECODE_WAVES waves per workgroup.  The macro tiles of a split go round-robin to
// the waves (operands straight from global memory: all of a macro tile's loads are in flight together), which
// combine their running softmax states through LDS.  With one split the workgroup writes the output itself;
// with several it writes a partial (max, sum, unnormalised output) per head, and the merge kernel below
// combines the partials with the log-sum-exp rule.  (Merging inside this kernel, by the workgroup that
// finishes last, was measured: the device-wide fences it needs cost many times the second launch.)
// Partials: part_o [entries, nq, num_splits, D], part_ml [entries, nq, num_splits, 2] (max in base-2 units).
// A launch whose key ranges make two such workgroups or more for every compute unit runs with workgroups of twice
// the waves and half the ranges instead (WAVES = DECODE_WAVES_WIDE): half as many workgroups to hand out, fewer
// heads a wave for the norms and the rotation, half the partials for the merge (8 requests of 2,048 tokens: 19.1
// against 20.5 us with the merge, 16 requests 30.0 against 32.7; one request, whose 64 workgroups are few enough
// already, 12.8 against 11.5, so the caller says which).
constexpr int DECODE_WAVES = D > 128 ? 2 : 4;
constexpr int DECODE_WAVES_WIDE = 2 * DECODE_WAVES;

// With FRONT, the kernel also does what precedes attention for a decoded token (fused_qwen3.py:98-107 of the
// reference): `q` is then the raw fused projection [tokens, (nq + 2 nkv) D] with rows q | k | v.  Every workgroup
// norms and rotates its group's queries into LDS; the new key is normed and rotated there too.  The cached keys
// are those before the new token; the new key and value enter the softmax from registers, in wave 0 of split 0,
// which also writes them to their cache slot for later steps.
struct DecodeFront {
  const float* q_weight;     // [D] or null: per-head RMS norm weights
  const float* k_weight;
  float eps;
  const float* cos_sin;      // [max_pos, rotary_dim] or null
  int rotary_dim;
  int max_pos;
  const int* positions;      // [tokens]
  const int* slots;          // [tokens] slot of each token's key and value: page * P + offset
  uint16_t* k_pages;
  uint16_t* v_pages;
};

__device__ __forceinline__ float bf16_at(const uint16_t* p) { return __uint_as_float((uint32_t)(*p) << 16); }

template <bool FRONT, bool STREAM, int WAVES>
__global__ __launch_bounds__(64 * WAVES) DECODE_OCCUPANCY void decode_kernel(
    const uint16_t* __restrict__ q, int64_t q_row_stride, uint16_t* __restrict__ out, int64_t out_row_stride,
    const uint16_t* __restrict__ k_pages, const uint16_t* __restrict__ v_pages, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ cu_q, const int* __restrict__ kv_len, int first_entry,
    float* __restrict__ part_o, float* __restrict__ part_ml, int nq, int nkv, int page_shift, float scale,
    int window, DecodeFront front) {
  __shared__ float lds_o[WAVES][DBLK][64][4];
  __shared__ float lds_m[WAVES][16];
  __shared__ float lds_l[WAVES][16];
  __shared__ __attribute__((aligned(16))) uint16_t lds_q[FRONT ? 16 * D : 8];   // normed, rotated queries of the group
  __shared__ __attribute__((aligned(16))) uint16_t lds_k[FRONT ? D : 8];        // and the new key
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int split = blockIdx.x, num_splits = gridDim.x;
  const int g = blockIdx.y;
  const int e = blockIdx.z;             // entry index among the decode entries
  const int b = first_entry + e;
  const int G = nq / nkv;
  const int P = 1 << page_shift;
  const int kv = kv_len[b];
  const int pos = kv - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int last = FRONT ? pos - 1 : pos;   // last key that is read from the cache
  // this split's keys: macro tiles from the first visible one, evenly over the splits
  const int tile_lo = lo / MKEYS, tile_hi = last < lo ? tile_lo : last / MKEYS + 1;
  const int tiles_per_split = (tile_hi - tile_lo + num_splits - 1) / num_splits;
  const int t0 = tile_lo + split * tiles_per_split;
  const int t1 = min(tile_hi, t0 + tiles_per_split);
  const int* bt = block_table + (int64_t)b * table_width;
  const float c = scale * 1.44269504088896340736f;
  const int token = cu_q[b];

  // STREAM: the launch's keys and values are many times what the caches hold and are read once a step; nontemporal
  // loads keep them from pushing everything else out (64 requests of 2,048 tokens: 87 against 99 us a layer, 6.15
  // against 5.44 TB/s; 8 requests of 32,768: 178 against 194 us).  Few keys are quicker with ordinary loads inside
  // a step (8 requests of 2,048: 17.9 against 18.5 us), so the caller says which.
  // the first macro tile's loads go out before anything else: nothing below depends on them until the products
  bf16x8 ka[MT][QSTEPS];
  s16x4 va[MT][DBLK];
#define DECODE_FETCH(TILE)                                                                                           \
  {                                                                                                                  \
    const int j0_ = (TILE) * MKEYS;                                                                                  \
    _Pragma("unroll") for (int t = 0; t < MT; ++t) { /* clamped addresses: masked keys read valid memory */         \
      int kk = j0_ + 16 * t + (lane & 15);                                                                           \
      kk = kk > pos ? pos : kk;                                                                                      \
      const int64_t kpage = bt[kk >> page_shift];                                                                    \
      if (STREAM) load_row_stream(ka[t], k_pages + ((kpage * nkv + g) * P + (kk & (P - 1))) * D);                    \
      else load_row(ka[t], k_pages + ((kpage * nkv + g) * P + (kk & (P - 1))) * D, true);                            \
      int vk = j0_ + 16 * t + 4 * (lane >> 4);                                                                       \
      vk = vk > pos ? (pos & ~3) : vk;                                                                               \
      const int64_t vpage = bt[vk >> page_shift];                                                                    \
      const uint16_t* vbase = v_pages + ((vpage * nkv + g) * D + (lane & 15)) * P + (vk & (P - 1));                  \
      _Pragma("unroll") for (int blk = 0; blk < DBLK; ++blk)                                                         \
          va[t][blk] = STREAM ? __builtin_nontemporal_load(reinterpret_cast<const s16x4*>(vbase + (int64_t)16 * blk * P)) \
                              : *reinterpret_cast<const s16x4*>(vbase + (int64_t)16 * blk * P);                       \
    }                                                                                                                \
  }
  int mt = t0 + wave;
  State<1> st;
  init_state<1>(st);
  const bool col_ok = (lane & 15) < G;
  QRegs qr[1];
  if constexpr (FRONT) {
    // Vector loads come back in the order they were issued, and the compiler can only wait for some of them in
    // straight-line code.  So everything the norm and the rotation read is asked for first, without branches
    // (absent operands read a stand-in address and are replaced afterwards), in two dependent rounds (the
    // position, then its angles); the first macro tile is asked for after that, and the arithmetic runs while the
    // tile is on its way.  Wave w takes heads w, w + WAVES, ... of the group's query heads followed by
    // its key head; a lane takes the rotation pairs (j, j + D/2), j = lane + 64 c.  Without a rotation table
    // the pairs are "rotated" by the angle 0.
    constexpr int HPW = (17 + WAVES - 1) / WAVES;
    constexpr int HALF = D / 2;
    constexpr int NP = (HALF + 63) / 64;
    const uint16_t* row = q + (int64_t)token * q_row_stride;
    const float* stand_in = reinterpret_cast<const float*>(row);      // at least D readable floats
    const bool has_rope = front.cos_sin != nullptr, has_qw = front.q_weight != nullptr,
               has_kw = front.k_weight != nullptr;
    int rp = *(has_rope ? front.positions + token : cu_q + b);
    float xa[HPW][NP], xb[HPW][NP];
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int hh = wave + WAVES * i;
      const uint16_t* src = row + (int64_t)(hh < G ? g * G + hh : nq + g) * D;
#pragma unroll
      for (int cc = 0; cc < NP; ++cc) {
        const int j = min(lane + 64 * cc, HALF - 1);
        xa[i][cc] = bf16_at(src + j);
        xb[i][cc] = bf16_at(src + j + HALF);
      }
    }
    float wqa[NP], wqb[NP], wka[NP], wkb[NP], cva[NP], sva[NP];
    const float* qwp = has_qw ? front.q_weight : stand_in;
    const float* kwp = has_kw ? front.k_weight : stand_in;
#pragma unroll
    for (int cc = 0; cc < NP; ++cc) {
      const int j = min(lane + 64 * cc, HALF - 1);
      wqa[cc] = qwp[j];
      wqb[cc] = qwp[j + HALF];
      wka[cc] = kwp[j];
      wkb[cc] = kwp[j + HALF];
    }
    rp = rp < 0 ? 0 : (rp >= front.max_pos ? front.max_pos - 1 : rp);
    const float* cs = has_rope ? front.cos_sin + (int64_t)rp * D : stand_in;
#pragma unroll
    for (int cc = 0; cc < NP; ++cc) {
      const int j = min(lane + 64 * cc, HALF - 1);
      cva[cc] = cs[j];
      sva[cc] = cs[HALF + j];
    }
    DECODE_FETCH(min(mt, max(t1 - 1, t0)))      // a wave without a tile asks for one all the same and drops it
#pragma unroll
    for (int cc = 0; cc < NP; ++cc) {
      if (!has_qw) wqa[cc] = wqb[cc] = 1.f;
      if (!has_kw) wka[cc] = wkb[cc] = 1.f;
      if (!has_rope) {
        cva[cc] = 1.f;
        sva[cc] = 0.f;
      }
    }
#pragma unroll
    for (int i = 0; i < HPW; ++i) {
      const int hh = wave + WAVES * i;
      if (hh <= G) {                           // the same for every lane of the wave
        const bool is_key = hh == G;
        uint16_t* dst = is_key ? lds_k : lds_q + hh * D;
        float ss = 0.f;
#pragma unroll
        for (int cc = 0; cc < NP; ++cc)
          if (lane + 64 * cc < HALF) ss += xa[i][cc] * xa[i][cc] + xb[i][cc] * xb[i][cc];
        const float rstd = (is_key ? has_kw : has_qw) ? rsqrtf(wave_sum(ss) / (float)D + front.eps) : 1.f;
#pragma unroll
        for (int cc = 0; cc < NP; ++cc) {
          const int j = lane + 64 * cc;
          if (j < HALF) {
            const float a = xa[i][cc] * rstd * (is_key ? wka[cc] : wqa[cc]);
            const float b2 = xb[i][cc] * rstd * (is_key ? wkb[cc] : wqb[cc]);
            dst[j] = float_to_bf16_bits(a * cva[cc] - b2 * sva[cc]);
            dst[j + HALF] = float_to_bf16_bits(b2 * cva[cc] + a * sva[cc]);
          }
        }
      }
    }
    __syncthreads();
    load_queries<1>(qr, lds_q, D, 16, G, 1, 0);
  } else {
    load_queries<1>(qr, q + (int64_t)token * q_row_stride, q_row_stride, 16, G, 1, g * G);
    if (mt < t1) DECODE_FETCH(mt)
  }
  const int pos_lo[1] = {lo};
  const int pos_hi[1] = {col_ok ? last : -1};
  while (mt < t1) {
    const int j0 = mt * MKEYS;
    f32x4 s[MT][1];
    s16x4 p[MT][1];
#pragma unroll
    for (int t = 0; t < MT; ++t) tile_scores<1>(s[t], ka[t], qr);
    softmax_update<1>(st, s, p, c, j0, pos_lo, pos_hi);
#pragma unroll
    for (int t = 0; t < MT; t += 2) tile_values<1>(st, va[t], va[t + 1], p[t], p[t + 1]);
    mt += WAVES;
    if (mt < t1) DECODE_FETCH(mt)
  }
#undef DECODE_FETCH
  if constexpr (FRONT) {
    if (split == 0 && wave == 0) {
      // the new token's own key and value: one more softmax step, from LDS and the projection's row
      bf16x8 kn[QSTEPS];
      load_row(kn, lds_k, true);
      float dot = 0.f;
#pragma unroll
      for (int ks = 0; ks < QSTEPS; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) dot += (float)qr[0].full[ks][i] * (float)kn[ks][i];
      dot += __shfl_xor(dot, 16, 64);
      dot += __shfl_xor(dot, 32, 64);
      const float v = col_ok ? dot * c : -INFINITY;
      const float m_new = fmaxf(st.m[0], v);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f(st.m[0] - m_use);
      const float pe = __builtin_amdgcn_exp2f(v - m_use);
      const float pr = __uint_as_float((uint32_t)float_to_bf16_bits(pe) << 16);   // rounded like the tiles' P
      st.l[0] = st.l[0] * alpha + ((lane >> 4) == 0 ? pe : 0.f);
      st.m[0] = m_new;
      const uint16_t* vrow = q + (int64_t)token * q_row_stride + (int64_t)(nq + nkv + g) * D;
      const int slot = front.slots[token];
      const int64_t page = slot >> page_shift;
      const int off = slot & (P - 1);
#pragma unroll
      for (int blk = 0; blk < DBLK; ++blk) {
        const s16x4 vv = *reinterpret_cast<const s16x4*>(vrow + 16 * blk + 4 * (lane >> 4));
#pragma unroll
        for (int i = 0; i < 4; ++i)
          st.o[0][blk][i] = st.o[0][blk][i] * alpha + pr * __uint_as_float((uint32_t)(uint16_t)vv[i] << 16);
      }
      // the cache copies: the key's row, and the value's elements into the transposed page
      uint16_t* kdst = front.k_pages + ((page * nkv + g) * P + off) * D;
      uint16_t* vdst = front.v_pages + (page * nkv + g) * (int64_t)D * P + off;
      for (int i = lane; i < D; i += 64) {
        kdst[i] = lds_k[i];
        vdst[(int64_t)i * P] = vrow[i];
      }
    }
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
  // thread -> (block of dims, lane slot): column col = slot % 16, dims 16 blk + 4 (slot / 16) + i
  for (int idx = threadIdx.x; idx < DBLK * 64; idx += blockDim.x) {
    const int blk = idx >> 6, slot = idx & 63;
    const int col = slot & 15;
    if (col >= G) continue;
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) M = fmaxf(M, lds_m[w][col]);
    f32x4 acc = {0.f, 0.f, 0.f, 0.f};
    float L = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float mw = lds_m[w][col];
      const float wt = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - M);
      const f32x4 v = *reinterpret_cast<const f32x4*>(&lds_o[w][blk][slot][0]);
      acc[0] += wt * v[0];
      acc[1] += wt * v[1];
      acc[2] += wt * v[2];
      acc[3] += wt * v[3];
      L += wt * lds_l[w][col];
    }
    const int head = g * G + col;
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

// Up to FEW splits of one (entry, head): everything is asked for at once, the partial outputs before the maxima
// and sums that weigh them are known, so the wave waits for memory once.  A lane takes 4 dims and reads every
// split's (max, sum) itself.
template <int FEW>
__device__ __forceinline__ void merge_few(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                          int64_t base, int num_splits, uint16_t* __restrict__ o) {
  static_assert(D <= 256, "a lane takes 4 of at most 256 dims");
  const int lane = threadIdx.x;
  const bool live = 4 * lane < D;
  const int d0 = live ? 4 * lane : 0;
  float2 ml[FEW];
  f32x4 v[FEW];
#pragma unroll
  for (int j = 0; j < FEW; ++j) {
    const int jj = j < num_splits ? j : num_splits - 1;        // a split again instead of a branch
    ml[j] = *reinterpret_cast<const float2*>(part_ml + (base + jj) * 2);
    v[j] = *reinterpret_cast<const f32x4*>(part_o + (base + jj) * D + d0);
  }
  float M = -INFINITY;
#pragma unroll
  for (int j = 0; j < FEW; ++j) M = fmaxf(M, ml[j].x);
  float L = 0.f;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int j = 0; j < FEW; ++j) {
    const float w = (j < num_splits && ml[j].x != -INFINITY) ? __builtin_amdgcn_exp2f(ml[j].x - M) : 0.f;
    L += w * ml[j].y;
    acc[0] += w * v[j][0];
    acc[1] += w * v[j][1];
    acc[2] += w * v[j][2];
    acc[3] += w * v[j][3];
  }
  const float inv = 1.f / L;
  if (live) *reinterpret_cast<s16x4*>(o + d0) = pack_bf16x4(acc[0] * inv, acc[1] * inv, acc[2] * inv, acc[3] * inv);
}

// out[token of entry e][head] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s
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
  if (num_splits <= 32) {
    uint16_t* o = out + (int64_t)cu_q[first_entry + e] * out_row_stride + (int64_t)head * D;
    if (num_splits <= 8) merge_few<8>(part_o, part_ml, base, num_splits, o);
    else if (num_splits <= 16) merge_few<16>(part_o, part_ml, base, num_splits, o);
    else merge_few<32>(part_o, part_ml, base, num_splits, o);
    return;
  }
  constexpr int MAXR = 16;                       // 64 * 16 = 1024 splits at most
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
    mv[r] = (mv[r] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mv[r] - M);   // now the split's weight
    L += mv[r] * lv[r];
    if (64 * (r + 1) >= num_splits) break;
  }
  L = wave_sum(L);
  const float inv = 1.f / L;
  uint16_t* o = out + (int64_t)cu_q[first_entry + e] * out_row_stride + (int64_t)head * D;
  // dims: 4 per lane and round; every lane runs every round (the shuffles below need all lanes)
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

// The same for more than 32 splits (one long request: the key ranges then outnumber what a wave's loads cover at
// once): a workgroup of 4 waves per (entry, head).  The threads share out the splits for the maximum and the weights,
// which are kept in LDS; then thread (group, 4 dims) adds the splits group, group + G, ... of its dims, whose loads do
// not depend on one another, and the groups' sums are added in order.
__global__ __launch_bounds__(256) void decode_merge_many_kernel(const float* __restrict__ part_o,
                                                               const float* __restrict__ part_ml,
                                                               uint16_t* __restrict__ out, int64_t out_row_stride,
                                                               const int* __restrict__ cu_q, int first_entry, int nq,
                                                               int num_splits) {
  __shared__ float wts[1024];
  __shared__ float red4[4];
  __shared__ f32x4 accs[256];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int e = blockIdx.x / nq, head = blockIdx.x % nq;
  const int64_t base = ((int64_t)e * nq + head) * num_splits;
  float M = -INFINITY;
  for (int s = tid; s < num_splits; s += 256) M = fmaxf(M, part_ml[(base + s) * 2]);
  M = wave_max(M);
  if (lane == 0) red4[wave] = M;
  __syncthreads();
  M = fmaxf(fmaxf(red4[0], red4[1]), fmaxf(red4[2], red4[3]));
  __syncthreads();
  float L = 0.f;
  for (int s = tid; s < num_splits; s += 256) {
    const float2 ml = *reinterpret_cast<const float2*>(part_ml + (base + s) * 2);
    const float w = ml.x == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(ml.x - M);
    wts[s] = w;
    L += w * ml.y;
  }
  L = wave_sum(L);
  if (lane == 0) red4[wave] = L;
  __syncthreads();
  L = (red4[0] + red4[1]) + (red4[2] + red4[3]);
  constexpr int DL = D / 4 <= 4 ? 4 : (D / 4 <= 8 ? 8 : (D / 4 <= 16 ? 16 : (D / 4 <= 32 ? 32 : 64)));
  constexpr int G = 256 / DL;
  const int grp = tid / DL, dl = tid % DL;
  const bool live = 4 * dl < D;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (live) {
    const float* po = part_o + base * D + 4 * dl;
#pragma unroll 8
    for (int s = grp; s < num_splits; s += G) {
      const f32x4 v = *reinterpret_cast<const f32x4*>(po + (int64_t)s * D);
      const float w = wts[s];
      acc[0] += w * v[0];
      acc[1] += w * v[1];
      acc[2] += w * v[2];
      acc[3] += w * v[3];
    }
  }
  accs[tid] = acc;
  __syncthreads();
  if (grp == 0 && live) {
    f32x4 t = accs[dl];
    for (int g2 = 1; g2 < G; ++g2) {
      const f32x4 v = accs[g2 * DL + dl];
      t[0] += v[0];
      t[1] += v[1];
      t[2] += v[2];
      t[3] += v[3];
    }
    const float inv = 1.f / L;
    uint16_t* o = out + (int64_t)cu_q[first_entry + e] * out_row_stride + (int64_t)head * D;
    *reinterpret_cast<s16x4*>(o + 4 * dl) = pack_bf16x4(t[0] * inv, t[1] * inv, t[2] * inv, t[3] * inv);
  }
}

static void launch_decode_merge(const float* part_o, const float* part_ml, uint16_t* out, int64_t out_row_stride,
                                const int* cu_q, int first_entry, int num_entries, int nq, int num_splits,
                                hipStream_t stream) {
  if (num_splits > 32)
    decode_merge_many_kernel<<<num_entries * nq, 256, 0, stream>>>(part_o, part_ml, out, out_row_stride, cu_q,
                                                                  first_entry, nq, num_splits);
  else
    decode_merge_kernel<<<num_entries * nq, 64, 0, stream>>>(part_o, part_ml, out, out_row_stride, cu_q, first_entry,
                                                             nq, num_splits);
}

// ---------------------------------------------------------------- entry points
static int check_common(const char* what, int nq, int nkv, int page_size, int64_t q_row_stride, int64_t out_row_stride,
                        int table_width) {
  MI_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "%s: %d query heads are no multiple of %d kv heads", what, nq, nkv);
  MI_REQUIRE(nq / nkv <= 16, "%s: %d query heads per kv head; this kernel takes at most 16", what, nq / nkv);
  MI_REQUIRE(page_size >= 8 && (page_size & (page_size - 1)) == 0, "%s: page size %d is not a power of two >= 8", what,
             page_size);
  MI_REQUIRE(q_row_stride >= (int64_t)nq * D && q_row_stride % 8 == 0, "%s: query row stride %lld", what,
             (long long)q_row_stride);
  MI_REQUIRE(out_row_stride >= (int64_t)nq * D && out_row_stride % 4 == 0, "%s: output row stride %lld", what,
             (long long)out_row_stride);
  MI_REQUIRE(table_width > 0, "%s: empty block table", what);
  return 0;
}

static int check_scale(const char* what, float scale) {
  MI_REQUIRE(scale > 0.f, "%s: the softmax scale must be positive, got %g", what, (double)scale);
  return 0;
}

static int log2_of(int v) {
  int s = 0;
  while ((1 << s) < v) ++s;
  return s;
}

static int group_pad(int nq, int nkv) {
  int gpad = 1;
  while (gpad < nq / nkv) gpad <<= 1;
  return gpad;
}

MI_EXPORT int mi_attn_head_dim() { return D; }

// Keys per macro tile: the granule of the decode kernel's key splits.
MI_EXPORT int mi_attn_macro_tile_keys() { return MKEYS; }

// Waves per workgroup of the decode kernel.
MI_EXPORT int mi_attn_decode_waves() { return DECODE_WAVES; }
MI_EXPORT int mi_attn_decode_waves_wide() { return DECODE_WAVES_WIDE; }

// Query tokens per work item (a workgroup of 4 waves, 16 * PREFILL_NB columns each) of the prefill launch.
MI_EXPORT int mi_attn_prefill_tokens_per_block(int nq, int nkv) {
  const int gpad = group_pad(nq, nkv);
  return gpad > 16 ? 0 : 4 * (16 * PREFILL_NB / gpad);
}

// The same for the instance with two column blocks per wave (variant 3 of mi_attn_prefill); 0 where there is none.
MI_EXPORT int mi_attn_prefill_tokens_per_block_wide(int nq, int nkv) {
  const int gpad = group_pad(nq, nkv);
  return (gpad > 16 || !PREFILL_WIDE) ? 0 : 4 * (32 / gpad);
}

MI_EXPORT int mi_attn_prefill(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride, const void* k_pages,
                              const void* v_pages, const int* block_table, int table_width, const int* work,
                              int num_work, const int* cu_q, const int* kv_len, int nq, int nkv, int page_size,
                              float scale, int window, int variant, hipStream_t stream) {
  // variant: 0 = chosen from the grid's size; 1 = 8 waves, two macro tiles a step; 2 = 4 waves, three waves a SIMD;
  // 3 = 4 waves with two column blocks each (its work items count mi_attn_prefill_tokens_per_block_wide tokens)
  if (check_common("attn_prefill", nq, nkv, page_size, q_row_stride, out_row_stride, table_width)) return 1;
  MI_REQUIRE(variant >= 0 && variant <= 3, "attn_prefill: variant %d", variant);
  MI_REQUIRE(variant != 3 || PREFILL_WIDE, "attn_prefill: head size %d has no instance with two column blocks", D);
  if (check_scale("attn_prefill", scale)) return 1;
  MI_REQUIRE(num_work >= 0 && window >= 0, "attn_prefill: bad work count or window");
  MI_REQUIRE(num_work <= 65535, "attn_prefill: %d work items; the grid takes at most 65535", num_work);
  if (num_work == 0) return 0;
  dim3 grid(nkv, num_work);
  static int compute_units = 0;
  if (compute_units == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&compute_units, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
        compute_units <= 0)
      compute_units = 256;
  }
#if PREFILL_WIDE
  if (variant == 3) {
    prefill_wide_kernel<<<grid, 256, 0, stream>>>(
        (const uint16_t*)q, q_row_stride, (uint16_t*)out, out_row_stride, (const uint16_t*)k_pages,
        (const uint16_t*)v_pages, block_table, table_width, work, cu_q, kv_len, nq, nkv, group_pad(nq, nkv),
        log2_of(page_size), scale, window);
    MI_CHECK_LAUNCH("attn_prefill");
    return 0;
  }
#endif
  if (variant == 2 || (variant == 0 && (int64_t)num_work * nkv > 2 * (int64_t)compute_units))
    prefill_dense_kernel<PREFILL_NB><<<grid, 256, 0, stream>>>(
        (const uint16_t*)q, q_row_stride, (uint16_t*)out, out_row_stride, (const uint16_t*)k_pages,
        (const uint16_t*)v_pages, block_table, table_width, work, cu_q, kv_len, nq, nkv, group_pad(nq, nkv),
        log2_of(page_size), scale, window);
  else
    prefill_kernel<PREFILL_NB><<<grid, 512, 0, stream>>>(
        (const uint16_t*)q, q_row_stride, (uint16_t*)out, out_row_stride, (const uint16_t*)k_pages,
        (const uint16_t*)v_pages, block_table, table_width, work, cu_q, kv_len, nq, nkv, group_pad(nq, nkv),
        log2_of(page_size), scale, window);
  MI_CHECK_LAUNCH("attn_prefill");
  return 0;
}

// Entries first_entry .. first_entry + num_entries - 1 must each bring exactly one token.
// part_o: float [num_entries * nq * num_splits * D]; part_ml: float [num_entries * nq * num_splits * 2].
// stream_keys: read the keys and values with nontemporal loads (for launches that read many times the caches' size).
// wide: workgroups of mi_attn_decode_waves_wide() waves instead of mi_attn_decode_waves().
MI_EXPORT int mi_attn_decode(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride, const void* k_pages,
                             const void* v_pages, const int* block_table, int table_width, const int* cu_q,
                             const int* kv_len, int first_entry, int num_entries, int num_splits, float* part_o,
                             float* part_ml, int nq, int nkv, int page_size, float scale, int window,
                             int stream_keys, int wide, hipStream_t stream) {
  if (check_common("attn_decode", nq, nkv, page_size, q_row_stride, out_row_stride, table_width)) return 1;
  if (check_scale("attn_decode", scale)) return 1;
  MI_REQUIRE(num_entries >= 0 && first_entry >= 0 && window >= 0, "attn_decode: bad entry range or window");
  MI_REQUIRE(num_splits >= 1 && num_splits <= 1024, "attn_decode: %d splits", num_splits);
  MI_REQUIRE(num_entries <= 65535 && nkv <= 65535, "attn_decode: grid too large");
  MI_REQUIRE(num_splits == 1 || (part_o && part_ml), "attn_decode: no partial buffers");
  if (num_entries == 0) return 0;
  dim3 grid(num_splits, nkv, num_entries);
#define DECODE_GO_W(FRONT, STREAM, WV, Q, QS, F)                                                                   \
  decode_kernel<FRONT, STREAM, WV><<<grid, 64 * WV, 0, stream>>>(                                                   \
      (const uint16_t*)(Q), QS, (uint16_t*)out, out_row_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages, \
      block_table, table_width, cu_q, kv_len, first_entry, part_o, part_ml, nq, nkv, log2_of(page_size), scale,     \
      window, F)
#define DECODE_GO(FRONT, STREAM, Q, QS, F)                                                                          \
  {                                                                                                                  \
    if (wide) DECODE_GO_W(FRONT, STREAM, DECODE_WAVES_WIDE, Q, QS, F);                                               \
    else DECODE_GO_W(FRONT, STREAM, DECODE_WAVES, Q, QS, F);                                                         \
  }
  if (stream_keys) DECODE_GO(false, true, q, q_row_stride, DecodeFront{})
  else DECODE_GO(false, false, q, q_row_stride, DecodeFront{})
  MI_CHECK_LAUNCH("attn_decode");
  if (num_splits > 1) {
    launch_decode_merge(part_o, part_ml, (uint16_t*)out, out_row_stride, cu_q, first_entry, num_entries, nq, num_splits,
                        stream);
    MI_CHECK_LAUNCH("attn_decode merge");
  }
  return 0;
}

// The same for entries whose projection has not been normed, rotated or cached yet: qkv [tokens, >= (nq + 2 nkv) D]
// holds rows q | k | v of the fused projection; q_weight / k_weight [D] float32 or null; cos_sin [max_pos, rotary_dim]
// float32 or null; positions and slots per token.  The new keys and values are written to their slots.
MI_EXPORT int mi_attn_decode_front(const void* qkv, int64_t qkv_row_stride, void* out, int64_t out_row_stride,
                                   void* k_pages, void* v_pages, const int* block_table, int table_width,
                                   const int* cu_q, const int* kv_len, int first_entry, int num_entries, int num_splits,
                                   float* part_o, float* part_ml, int nq, int nkv, int page_size, float scale,
                                   int window, int stream_keys, int wide, const float* q_weight, const float* k_weight,
                                   float eps, const float* cos_sin, int rotary_dim, int max_pos,
                                   const int* positions, const int* slots, hipStream_t stream) {
  if (check_common("attn_decode_front", nq, nkv, page_size, qkv_row_stride, out_row_stride, table_width)) return 1;
  if (check_scale("attn_decode_front", scale)) return 1;
  MI_REQUIRE(qkv_row_stride >= (int64_t)(nq + 2 * nkv) * D, "attn_decode_front: row stride %lld holds no q | k | v",
             (long long)qkv_row_stride);
  MI_REQUIRE(num_entries >= 0 && first_entry >= 0 && window >= 0, "attn_decode_front: bad entry range or window");
  MI_REQUIRE(num_splits >= 1 && num_splits <= 1024, "attn_decode_front: %d splits", num_splits);
  MI_REQUIRE(num_entries <= 65535 && nkv <= 65535, "attn_decode_front: grid too large");
  MI_REQUIRE(num_splits == 1 || (part_o && part_ml), "attn_decode_front: no partial buffers");
  MI_REQUIRE(slots && k_pages && v_pages, "attn_decode_front: no cache slots");
  if (cos_sin)
    MI_REQUIRE(rotary_dim == D && positions && max_pos > 0,
               "attn_decode_front: rotary_dim %d; this kernel rotates whole heads of %d only", rotary_dim, D);
  if (num_entries == 0) return 0;
  DecodeFront front{q_weight, k_weight, eps, cos_sin, rotary_dim, max_pos, positions, slots, (uint16_t*)k_pages,
                    (uint16_t*)v_pages};
  dim3 grid(num_splits, nkv, num_entries);
  if (stream_keys) DECODE_GO(true, true, qkv, qkv_row_stride, front)
  else DECODE_GO(true, false, qkv, qkv_row_stride, front)
#undef DECODE_GO
#undef DECODE_GO_W
  MI_CHECK_LAUNCH("attn_decode_front");
  if (num_splits > 1) {
    launch_decode_merge(part_o, part_ml, (uint16_t*)out, out_row_stride, cu_q, first_entry, num_entries, nq, num_splits,
                        stream);
    MI_CHECK_LAUNCH("attn_decode_front merge");
  }
  return 0;
}

// ---------------------------------------------------------------- decode without a workspace argument
// The partials of the key splits in a device array of the shared object itself (see attention_mfma.h).
static __device__ __align__(256) float scratch[MI_ATTN_STATIC_SCRATCH_FLOATS];

// In host code `scratch` is only a handle of the symbol, never an address a kernel may use: each device has its own
// copy of the array at its own address, asked for once per device with that device current.
constexpr int STATIC_MAX_DEVICES = 64;
static float* g_scratch_ptr[STATIC_MAX_DEVICES] = {nullptr};
static std::mutex g_scratch_mutex;

static int static_scratch(float** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  MI_REQUIRE(e == hipSuccess, "attn_decode_static: hipGetDevice failed: %s", hipGetErrorString(e));
  MI_REQUIRE(dev >= 0 && dev < STATIC_MAX_DEVICES, "attn_decode_static: device %d; at most %d are served", dev,
             STATIC_MAX_DEVICES);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    MI_REQUIRE(e == hipSuccess && p != nullptr, "attn_decode_static: hipGetSymbolAddress failed on device %d: %s", dev,
               hipGetErrorString(e));
    g_scratch_ptr[dev] = static_cast<float*>(p);
  }
  *ptr = g_scratch_ptr[dev];
  return 0;
}

MI_EXPORT int mi_attn_static_scratch_floats() { return MI_ATTN_STATIC_SCRATCH_FLOATS; }

MI_EXPORT int mi_attn_decode_static(const void* q, int64_t q_row_stride, void* out, int64_t out_row_stride,
                                    const void* k_pages, const void* v_pages, const int* block_table, int table_width,
                                    const int* cu_q, const int* kv_len, int first_entry, int num_entries,
                                    int num_splits, int nq, int nkv, int page_size, float scale, int window,
                                    hipStream_t stream) {
  MI_REQUIRE(num_entries >= 0 && num_splits >= 1 && nq > 0, "attn_decode_static: bad entry range or splits");
  const int64_t need = (int64_t)num_entries * nq * num_splits;        // partials: D floats of output, 2 of (max, sum)
  // part_o first, part_ml behind it on the next 64-byte boundary (need * D is a multiple of 16 floats as long as the
  // head size is one; the rounding keeps the alignment whatever a later head size may be)
  const int64_t ml_offset = (need * D + 15) / 16 * 16;
  MI_REQUIRE(num_splits == 1 || ml_offset + 2 * need <= (int64_t)MI_ATTN_STATIC_SCRATCH_FLOATS,
             "attn_decode_static: %d entries x %d heads x %d splits need %lld floats of partial results; the static "
             "scratch holds %d (use fewer splits, or mi_attn_decode with a workspace of your own)",
             num_entries, nq, num_splits, (long long)(ml_offset + 2 * need), MI_ATTN_STATIC_SCRATCH_FLOATS);
  float* base = nullptr;
  if (static_scratch(&base)) return 1;
  return mi_attn_decode(q, q_row_stride, out, out_row_stride, k_pages, v_pages, block_table, table_width, cu_q, kv_len,
                        first_entry, num_entries, num_splits, base, base + ml_offset, nq, nkv, page_size, scale, window,
                        0, 0, stream);
}
