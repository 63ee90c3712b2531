// C[M, N] = A[M, K] * W[N, K]^T in bfloat16 for few rows of A (M <= 64): the decode step's projections
// and the output head, whose time is the time to stream W once from HBM.
//
// The product is computed transposed on the matrix cores, C^T[n, m] = W[n, :] . A[m, :], so that the
// 16 rows of an MFMA block are weight rows: each lane's operand slot holds 16 contiguous bytes of a weight row,
// read straight from global memory or (see the modes below) written into LDS by loads of whole memory lines, and
// the few rows of A (which stay in L2) fill the other operand.  A workgroup owns 16 * RB weight rows; its waves
// split K and add their partial blocks through LDS.  32-bit accumulation; the result is stored as bfloat16 or float32.
// A second form, further down, splits K across workgroups instead (for 17 to 64 rows of A, where reading all of A
// in every workgroup is what the first form's time grows with); mi_gemm_skinny_v takes either.
//
// With GATE_UP, W is a fused gate|up matrix [2 N, K] (gate rows first) and the result is the feed-forward's
// activation C[m, n] = silu(A W_gate^T)[m, n] * (A W_up^T)[m, n] (kernels/triton/silu_mul.py:33-37 of the
// reference), made from the 32-bit sums of gate row n and up row n, which the same workgroup owns.
#include "common.h"
// SKINNY_NT: a second build of this file whose loads of W are nontemporal, for matrices that are read once a step
// and are larger than what the caches keep until the next step (the caller chooses the build by the matrix's size).
#ifdef SKINNY_NT
#define W_LOAD(PTR) __builtin_nontemporal_load(PTR)
#define W_LDS_AUX 2
#else
#define W_LOAD(PTR) (*(PTR))
#define W_LDS_AUX 0
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));   // (arrays of HIP's uint4 / float4 classes end up in scratch memory)

__device__ __forceinline__ bf16x8 zero_bf16x8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ float silu_f(float g) { return g / (1.f + expf(-g)); }

// Two optional halves of an RMS norm that sits between two products, so that the norm needs no kernel of its own.
// After the first product (`residual` set): instead of C, the workgroup adds its result to the 32-bit residual
// stream in place, r[m][n] += result, writes the next product's left operand a_out[m][n] = bf16(r[m][n] * w[n]),
// and the sum of r[m][n]^2 over its own columns n to ss_out[blockIdx.x][m] (rows of SS_ROW(M) entries: 16 when
// there are at most 16 rows, so that many small workgroups do not leave the next kernel a long table to read).
// Before the second product's result is stored (`row_ss` set): row m is scaled by rsqrt(sum_p row_ss[p][m] / K +
// eps), the norm's missing factor (K, the length of the normed rows, is this product's K).
#define SS_ROW(rows) ((rows) <= 16 ? 16 : 64)
#define SKINNY_CH(mb) ((mb) == 1 ? 8 : ((mb) == 2 ? 4 : 2))   // steps of K whose loads are asked for together
// KB of LDS in which a wave stages a chunk of the left operand: 16 mb rows of 4 CH pieces of 16 bytes
#define SKINNY_STAGE_KB(mb) ((mb) * SKINNY_CH(mb))
// The mode that stages both operands: steps per chunk, and KB for 16 blocks rows of 4 steps each
#define SKINNY_STAGE5_STEPS 4
#define SKINNY_STAGE5_KB(blocks) (16 * (blocks) * 4 * SKINNY_STAGE5_STEPS / 64)
struct NormHalves {
  const float* row_ss;      // [ss_parts][SS_ROW(M)]
  int ss_parts;
  float eps;
  float* residual;          // [M, N] float32, leading dimension N
  const float* norm_weight; // [N]
  uint16_t* a_out;          // [M, N] bfloat16, leading dimension N
  float* ss_out;            // [gridDim.x][SS_ROW(M)]
  int ss_stride;            // floats from one part's row of row_ss / ss_out to the next: SS_ROW(M)
};

// MODE 0 takes every shape.  MODES 1 to 5 are the same product for K a multiple of 32 and operands below 4 GB: the
// wave's number is made a scalar (its k range and every test on it then cost scalar instructions), addresses are a
// scalar base plus one 32-bit lane offset plus a constant, no load is masked (lanes of rows past the end read a live
// row again; their results are dropped at the end as before), and a wave's first weight loads go out before the
// index work of the norm halves' loads and of the staging below: what a unit's 16 waves do before their first
// loads is time added to the kernel (a hundred vector instructions each: 0.4 us), what they do after them is not.
// MODES 2 and 4: the left operand comes through LDS.  Straight from memory, an operand load takes 16 bytes per lane
// from 16 rows of A, half a memory line from each, and every workgroup reads all of A that way.  Instead a wave asks
// for its columns of A in runs that are contiguous in each row, has them written straight into its own piece of
// LDS (global_load_lds: lane i's 16 bytes land at base + 16 i), and takes the operands from there.  The staging
// pieces lie where the sums are added later.
// MODES 3 and 4 (K a multiple of 64): the weights come in whole memory lines too, two steps of k per pair of loads
// (see the loop).  MODE 5 (up to 16 rows of A): both operands come through LDS (see its block).  Modes 1, 2 and 5
// add the same products in the same order, and so do 3 and 4.
template <int MB, int RB, bool OUT_F32, bool GATE_UP, int MODE>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(const uint16_t* __restrict__ A, int64_t lda,
                                                           const uint16_t* __restrict__ W, int64_t ldw,
                                                           void* __restrict__ C, int64_t ldc, int M, int N, int K,
                                                           int rpg, NormHalves nh) {
  extern __shared__ float red[];   // [(waves + 1) / 2][RB * MB][256], then (norm halves) [OB * 256] squares, [waves][64] sums
  // A launch whose grid has a second dimension shares out the rows of A as well: workgroup (x, y) takes rows
  // 16 MB y .. of A (and of the result) against its rows of W, so that few rows of W still make workgroups enough;
  // the workgroups of one x read the same rows of W, and they are neighbours modulo 8 in launch order whenever the
  // grid's first dimension is a multiple of 8, that is on one XCD, whose L2 then holds those rows.
  const int m_base = 16 * MB * blockIdx.y;
  A += (int64_t)m_base * lda;
  M = min(M - m_base, 16 * MB);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);     // the same in every lane: said so
  const int nw = blockDim.x >> 6;
  // GATE_UP: RB == 2, row block 0 = gate rows n0.., row block 1 = up rows N + n0..; N counts output columns
  // rpg: rows of W per workgroup and row block: 16, or fewer so that the workgroups fill whole rounds of the
  // compute units (the lanes of the other rows then load nothing and their results are dropped).  Row block rb
  // starts at row n0 + rb * rpg (GATE_UP: at n0 of its half).
  constexpr int BLOCKS = GATE_UP ? 1 : RB;        // row blocks side by side in the result
  const int n0 = blockIdx.x * rpg * BLOCKS;
  const int n_end = min(N, n0 + rpg * BLOCKS);
  const bool w_live = (lane & 15) < rpg;
  constexpr bool WL = MODE == 3 || MODE == 4;     // weights fetched in whole memory lines (see below)
  constexpr bool STAGED = MODE == 2 || MODE == 4; // left operand through LDS
  const int steps = (K + 31) / 32;
  // steps of K per wave; with WL a wave's range is a whole number of pairs of steps (K is a multiple of 64 then)
  const int spw = WL ? 2 * ((steps / 2 + nw - 1) / nw) : (steps + nw - 1) / nw;
  const int s_begin = wave * spw;
  const int s_end = min(steps, s_begin + spw);

  f32x4 acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const uint16_t* wrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    int row = GATE_UP ? n0 + (lane & 15) : n0 + rpg * rb + (lane & 15);
    row = row < N ? row : N - 1;            // rows past the end read the last row; they are never stored
    if (GATE_UP && rb == 1) row += N;
    wrow[rb] = W + (int64_t)row * ldw;
  }
  const uint16_t* arow[MB];
  bool mok[MB];
#pragma unroll
  for (int mb = 0; mb < MB; ++mb) {
    const int m = 16 * mb + (lane & 15);
    mok[mb] = m < M;
    arow[mb] = A + (int64_t)(mok[mb] ? m : 0) * lda;
  }

  // What the norm halves read is asked for early, so that the end of the kernel does not wait for memory again:
  // the partial sums of squares of row (thread % SS), parts (thread / SS), + threads / SS, ... (four loads at a
  // time, added in the order of the parts); and the residual and norm weight of the first two result elements
  // this thread will finish.  MODE 0 asks before the weights; the other modes right after a wave's first weight
  // loads, which are what the kernel's time hangs on.
  constexpr int OBLK = GATE_UP ? MB : RB * MB;
  constexpr int SS = SS_ROW(16 * MB);
  float my_ss = 0.f;
  float r_pre[2] = {0.f, 0.f}, w_pre[2] = {0.f, 0.f};
#define SKINNY_NORM_PREFETCH()                                                                                       \
  {                                                                                                                  \
    int tid = threadIdx.x;                                                                                           \
    if (MODE != 0) asm volatile("" : "+v"(tid)); /* keeps the compiler from moving the index work in front of the loop */ \
    if (nh.row_ss) {                                                                                                 \
      const int m = tid % SS, stride = blockDim.x / SS;                                                            \
      for (int p = tid / SS; p < nh.ss_parts; p += 4 * stride) {                                                     \
        float v[4];                                                                                                  \
        _Pragma("unroll") for (int j = 0; j < 4; ++j)                                                                \
          v[j] = p + j * stride < nh.ss_parts ? nh.row_ss[(int64_t)(p + j * stride) * nh.ss_stride + m_base + m] : 0.f; \
        _Pragma("unroll") for (int j = 0; j < 4; ++j) my_ss += v[j];                                                 \
      }                                                                                                              \
    }                                                                                                                \
    if (nh.residual) {                                                                                               \
      _Pragma("unroll") for (int j = 0; j < 2; ++j) {                                                                \
        const int e = tid + j * blockDim.x;                                                                          \
        const int blk = e >> 8, ln = (e & 255) >> 2, i = e & 3;                                                      \
        const int r = 4 * (ln >> 4) + i; /* row within its block */                                                  \
        const int n = n0 + rpg * (blk / MB) + r;                                                                     \
        const int m = 16 * (blk % MB) + (ln & 15);                                                                   \
        if (e < OBLK * 256 && r < rpg && n < n_end && m < M) {                                                       \
          r_pre[j] = nh.residual[(int64_t)(m_base + m) * N + n];                                                     \
          w_pre[j] = nh.norm_weight[n];                                                                              \
        }                                                                                                            \
      }                                                                                                              \
    }                                                                                                                \
  }
  if constexpr (MODE == 0) SKINNY_NORM_PREFETCH()

  // Steps are taken CH at a time: first every load of the chunk is issued (weights, and the raw left operand),
  // then the operands are converted and multiplied, so one memory round trip covers CH steps.
  // what fits the 128 registers of a 16-wave workgroup (the exchange between lanes of the whole-line loads needs a
  // few registers more: two row blocks then take 4 steps at a time)
  constexpr int CH = (WL && RB == 2 && MB == 1) ? 4 : SKINNY_CH(MB);
  if constexpr (MODE == 0) {
    for (int s0 = s_begin; s0 < s_end; s0 += CH) {
      bf16x8 w[CH][RB];
      u32x4 ar[CH][MB];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        const int k = 32 * (s0 + c) + 8 * (lane >> 4);
        const bool kok = (s0 + c < s_end) && k < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
#pragma unroll
        for (int rb = 0; rb < RB; ++rb)
          w[c][rb] = (kok && w_live) ? W_LOAD(reinterpret_cast<const bf16x8*>(wrow[rb] + k)) : zero_bf16x8();
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          const bool ok = kok && mok[mb];
          ar[c][mb] = ok ? *reinterpret_cast<const u32x4*>(arow[mb] + k) : u32x4{0, 0, 0, 0};
        }
      }
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (s0 + c >= s_end) break;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) {
          union {
            u32x4 u;
            bf16x8 v;
          } a;
          a.u = ar[c][mb];
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[c][rb], a.v, acc[rb][mb], 0, 0, 0);
        }
      }
    }
  } else if constexpr (MODE == 5) {
    // Both operands through LDS (at most 16 rows of A).  Every request reads runs that are contiguous in a row, and
    // 16 lanes that are served together read one row's run: whole memory lines, the shape in which a large matrix
    // streams fastest (a bare read loop: 5.95 TB/s against 5.04 in the operand shape for [51200, 5120]).  Nothing
    // is held in registers meanwhile, so the chunks are short (4 steps: 16 pieces of 16 bytes per row) and the
    // waves many: what is in flight is what fits a compute unit's LDS.  Request f / 64, lane f % 64 fetches for the
    // place f % 16 of staged row f / 16 the piece (f % 16) ^ 2 (row % 4): an operand read (lanes l .. l + 3 with
    // l + 16 .. l + 19: 4 rows x 2 neighbouring pieces) then finds its 8 pieces in 8 different places (mod 8), that
    // is in different banks, without a byte of padding.
    static_assert(MB == 1, "this mode takes up to 16 rows of the left operand");
    constexpr int C5 = SKINNY_STAGE5_STEPS, ROWP = 4 * C5;
    static_assert(ROWP == 16, "the places of a row are swapped among 16");
    constexpr int NIW = SKINNY_STAGE5_KB(RB), NIA = SKINNY_STAGE5_KB(1);
    const int q = lane >> 4, r = lane & 15;
    // a wave's pieces: NIW KB for the weights, then as many KB as the M rows of the left operand need (rows past M
    // are read from whatever lies there; their results are dropped)
    const int kb_a = (M * ROWP + 63) / 64;
    uint16_t* stage_w = reinterpret_cast<uint16_t*>(red) + (size_t)wave * ((NIW + kb_a) * 512);
    uint16_t* stage_a = stage_w + NIW * 512;
    uint32_t w_off[NIW], a_off[NIA];
    int w_stp[NIW], a_stp[NIA];       // the step of the chunk a lane's piece belongs to; C5: never fetched
#pragma unroll
    for (int i = 0; i < NIW; ++i) {
      const int R = 4 * i + (lane >> 4);                // staged row; 16 lanes per row
      const int piece = (lane & 15) ^ (2 * (R & 3));
      int row = n0 + (GATE_UP ? 0 : rpg * (R >> 4)) + min(R & 15, rpg - 1);
      row = min(row, N - 1);
      if (GATE_UP && (R >> 4) == 1) row += N;
      w_off[i] = ((uint32_t)row * (uint32_t)ldw + 8 * piece) * 2;
      w_stp[i] = piece >> 2;
    }
    const char* wb = reinterpret_cast<const char*>(W) + (int64_t)s_begin * 64;
    const char* ab = reinterpret_cast<const char*>(A) + (int64_t)s_begin * 64;
    const int swz = 2 * (r & 3);                        // how this lane's row has its places swapped
    bool first = true;
    for (int left = s_end - s_begin; left > 0; left -= C5, wb += 64 * C5, ab += 64 * C5) {
      const int n = min(left, C5);                      // steps of this chunk: the same for the whole wave
#pragma unroll
      for (int i = 0; i < NIW; ++i)
        if (w_stp[i] < n)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wb + w_off[i]),
                                           (__attribute__((address_space(3))) void*)(stage_w + 512 * i), 16, 0, W_LDS_AUX);
      if (first) {
        first = false;
        SKINNY_NORM_PREFETCH()
        int lane_late = lane;
        asm volatile("" : "+v"(lane_late));             // keeps the compiler from moving this in front of the loop
#pragma unroll
        for (int i = 0; i < NIA; ++i) {
          const int R = 4 * i + (lane_late >> 4);
          const int piece = (lane_late & 15) ^ (2 * (R & 3));
          a_off[i] = R < M ? ((uint32_t)R * (uint32_t)lda + 8 * piece) * 2 : 0;
          a_stp[i] = R < M ? piece >> 2 : C5;
        }
      }
#pragma unroll
      for (int i = 0; i < NIA; ++i)
        if (a_stp[i] < n)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ab + a_off[i]),
                                           (__attribute__((address_space(3))) void*)(stage_a + 512 * i), 16, 0, 0);
      // The compiler does not count the requests that write LDS when it places the waits of the reads below: the
      // wait is written out, and nothing moves across it.
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
      for (int c = 0; c < C5; ++c) {
        if (c < n) {
          union {
            u32x4 u;
            bf16x8 v;
          } a, b;
          const int place = (4 * c + q) ^ swz;
          a.u = *reinterpret_cast<const u32x4*>(stage_a + 8 * (r * ROWP + place));
#pragma unroll
          for (int rb = 0; rb < RB; ++rb) {
            b.u = *reinterpret_cast<const u32x4*>(stage_w + 8 * ((16 * rb + r) * ROWP + place));
            acc[rb][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.v, a.v, acc[rb][0], 0, 0, 0);
          }
        }
      }
      // the reads above are done (their products have been issued) before the next chunk's requests overwrite them
      asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    if (first) SKINNY_NORM_PREFETCH()                   // a wave without a step of its own
    __syncthreads();                                    // the staging pieces are given up: the sums go where they were
  } else {
    const int q = lane >> 4, r = lane & 15;
    // byte offsets of the lane's 16 bytes in step 0 of the wave's range, from W + 64 s_begin and A + 64 s_begin
    // WL: an operand load as above takes 64 bytes from each of 16 rows, half a memory line; large matrices stream
    // a tenth to a sixth faster when every request is for whole lines.  So two steps are fetched together, by two
    // loads of 8 rows x 128 bytes: load i, lane (r, q) takes piece 2 q + r / 8 of row 8 i + r % 8.  Lanes r and
    // r + 8 then hold each other's data: the lower one its own row's even piece (load 0) and the other's (load 1),
    // the upper one the lower's odd piece and its own.  One rotation by 8 within the rows of 16 lanes
    // (update_dpp) puts both pieces of a row into its lane: piece 2 q serves the first step of the pair, 2 q + 1
    // the second; the left operand follows the same order of k.
    const int h = r >> 3, r8 = r & 7;
    uint32_t woff[RB][WL ? 2 : 1], aoff[MB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int i = 0; i < (WL ? 2 : 1); ++i) {
        int row = n0 + (GATE_UP ? 0 : rpg * rb) + min(WL ? 8 * i + r8 : r, rpg - 1);
        row = min(row, N - 1);
        if (GATE_UP && rb == 1) row += N;
        woff[rb][i] = ((uint32_t)row * (uint32_t)ldw + 8 * (WL ? 2 * q + h : q)) * 2;
      }
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
      aoff[mb] = ((uint32_t)min(16 * mb + r, M - 1) * (uint32_t)lda + (WL ? 16 : 8) * q) * 2;
    const char* wb = reinterpret_cast<const char*>(W) + (int64_t)s_begin * 64;
    const char* ab = reinterpret_cast<const char*>(A) + (int64_t)s_begin * 64;
    // MODE 2: the chunk's columns of A are rowp = 4 cs pieces of 16 bytes per row (cs: the steps of a wave's chunk
    // at most).  Request f / 64, lane f % 64 fetches piece f % rowp of row f / rowp, which lands at stage + 16 f
    // bytes.  (Rows padded to a stride that frees the operand reads of bank conflicts gained nothing here: these
    // few reads wait for the loads, not for LDS.)
    constexpr int NI = SKINNY_STAGE_KB(MB);             // requests per chunk at most
    uint16_t* stage = reinterpret_cast<uint16_t*>(red) + (size_t)wave * (NI * 512);
    const int rowp = 4 * min(CH, spw);
    uint32_t s_off[STAGED ? NI : 1];
    int s_stp[STAGED ? NI : 1];
    // (worked out after the first weight loads are on their way, like the norm halves' loads: a hundred vector
    // instructions in each of a unit's 16 waves before the first load cost the kernel 0.4 us)
#define SKINNY_STAGE_SETUP()                                                                                         \
  if constexpr (STAGED) {                                                                                            \
    int lane_late = lane;                                                                                            \
    asm volatile("" : "+v"(lane_late)); /* keeps the compiler from moving this in front of the loop */               \
    const uint32_t inv = (65536u + rowp - 1) / rowp; /* f / rowp = (f inv) >> 16 for f < 1024, rowp = 4 .. 32 */      \
    _Pragma("unroll") for (int i = 0; i < NI; ++i) {                                                                 \
      const int f = 64 * i + lane_late;                                                                              \
      const int row = (int)(((uint32_t)f * inv) >> 16), piece = f - row * rowp;                                      \
      const bool live = row < M;                                                                                     \
      s_off[i] = live ? ((uint32_t)row * (uint32_t)lda + 8 * piece) * 2 : 0;                                         \
      s_stp[i] = live ? piece >> 2 : CH; /* the step of the chunk it belongs to; CH: never fetched */                \
    }                                                                                                                \
  }
    bool first = true;
    for (int left = s_end - s_begin; left > 0; left -= CH, wb += 64 * CH, ab += 64 * CH) {
      const int n = min(left, CH);                      // steps of this chunk: the same for the whole wave
      u32x4 w[CH][RB];
      u32x4 ar[STAGED ? 1 : CH][MB];
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (c < n) {
#pragma unroll
          for (int rb = 0; rb < RB; ++rb)
            w[c][rb] = W_LOAD(reinterpret_cast<const u32x4*>(wb + woff[rb][WL ? c & 1 : 0] + (WL ? 128 * (c >> 1) : 64 * c)));
          if constexpr (!STAGED) {
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
              ar[c][mb] = *reinterpret_cast<const u32x4*>(ab + aoff[mb] + (WL ? 128 * (c >> 1) + 16 * (c & 1) : 64 * c));
          }
        }
      }
      if (first) {
        first = false;
        SKINNY_NORM_PREFETCH()
        SKINNY_STAGE_SETUP()
      }
      if constexpr (STAGED) {
#pragma unroll
        for (int i = 0; i < NI; ++i)
          if (s_stp[i] < n)
            __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(ab + s_off[i]),
                                             (__attribute__((address_space(3))) void*)(stage + 512 * i), 16, 0, 0);
        // The compiler does not count the requests that write LDS when it places the waits of the reads below:
        // the wait is written out, and nothing moves across it.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      }
      if constexpr (WL) {
        constexpr int ROR8 = 0x128;                     // row_ror:8
#pragma unroll
        for (int c = 0; c < CH; c += 2) {
          if (c < n) {
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
              const u32x4 l0 = w[c][rb], l1 = w[c + 1][rb];
#pragma unroll
              for (int e = 0; e < 4; ++e) {
                // lanes 8 .. 15 of a row take the lower lanes' load 1, lanes 0 .. 7 the upper lanes' load 0
                w[c][rb][e] = __builtin_amdgcn_update_dpp((int)l0[e], (int)l1[e], ROR8, 0xF, 0xC, false);
                w[c + 1][rb][e] = __builtin_amdgcn_update_dpp((int)l1[e], (int)l0[e], ROR8, 0xF, 0x3, false);
              }
            }
          }
        }
      }
#pragma unroll
      for (int c = 0; c < CH; ++c) {
        if (c < n) {
#pragma unroll
          for (int mb = 0; mb < MB; ++mb) {
            union {
              u32x4 u;
              bf16x8 v;
            } a, b;
            if constexpr (STAGED)
              a.u = *reinterpret_cast<const u32x4*>(
                  stage + 8 * ((16 * mb + r) * rowp + (WL ? 8 * (c >> 1) + 2 * q + (c & 1) : 4 * c + q)));
            else a.u = ar[c][mb];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) {
              b.u = w[c][rb];
              acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b.v, a.v, acc[rb][mb], 0, 0, 0);
            }
          }
        }
      }
    }
    if (first) SKINNY_NORM_PREFETCH()                   // a wave without a step of its own
    if constexpr (STAGED) __syncthreads();              // the staging pieces are given up: the sums go where they were
  }
#undef SKINNY_NORM_PREFETCH
#undef SKINNY_STAGE_SETUP

  // lane holds C^T[n0 + 16 rb + 4 (lane / 16) + i][16 mb + lane % 16].  The waves' blocks are added through LDS in
  // two rounds, which halves the LDS they need: the upper half of the waves leaves its blocks there, the lower
  // half adds them to its own (each lane the very words it holds) and leaves the sums; then the workgroup's
  // threads share out the elements of the result.
  constexpr int OB = GATE_UP ? MB : RB * MB;          // output blocks of the workgroup
  const int hw = (nw + 1) / 2;                        // waves whose sums stay in LDS
  float* sq = red + hw * RB * MB * 256;               // [OB * 256] squares of the new residual (norm halves only)
  float* ss_part = sq + OB * 256;                     // [waves][64]: each wave's sums by row
  if (wave >= hw) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        *reinterpret_cast<f32x4*>(red + (((wave - hw) * RB * MB + rb * MB + mb) * 64 + lane) * 4) = acc[rb][mb];
  }
  if (nh.row_ss) {
    if (SS == 16) {                                   // lanes l, l + 16, l + 32, l + 48 hold sums of the same row
      my_ss += __shfl_xor(my_ss, 16, 64);
      my_ss += __shfl_xor(my_ss, 32, 64);
    }
    ss_part[wave * 64 + lane] = my_ss;
  }
  __syncthreads();
  if (wave < hw) {
    const bool partner = wave + hw < nw;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        f32x4* p = reinterpret_cast<f32x4*>(red + ((wave * RB * MB + rb * MB + mb) * 64 + lane) * 4);
        *p = partner ? *p + acc[rb][mb] : acc[rb][mb];
      }
  }
  __syncthreads();
  // element e of the workgroup's result: block e / 256, lane (e % 256) / 4, register e % 4
  for (int e = threadIdx.x; e < OB * 256; e += blockDim.x) {
    const int blk = e >> 8, r = e & 255;
    float v = 0.f, u = 0.f;
    for (int w = 0; w < hw; ++w) {
      v += red[(w * RB * MB + blk) * 256 + r];
      if (GATE_UP) u += red[(w * RB * MB + MB + blk) * 256 + r];
    }
    const int ln = r >> 2, i = r & 3;
    const int rr = 4 * (ln >> 4) + i;             // row within its block
    const int n = n0 + rpg * (GATE_UP ? 0 : blk / MB) + rr;
    const int m = 16 * (blk % MB) + (ln & 15);
    if (nh.row_ss) {
      float total = 0.f;
      for (int w = 0; w < nw; ++w) total += ss_part[w * 64 + m];
      const float rstd = rsqrtf(total / (float)K + nh.eps);
      v *= rstd;
      u *= rstd;
    }
    if (GATE_UP) v = silu_f(v) * u;
    const bool live = rr < rpg && n < n_end && m < M;
    if (nh.residual) {
      float rv = 0.f;
      if (live) {
        const int j = (e - (int)threadIdx.x) / (int)blockDim.x;
        const float r_old = j == 0 ? r_pre[0] : (j == 1 ? r_pre[1] : nh.residual[(int64_t)(m_base + m) * N + n]);
        const float w_n = j == 0 ? w_pre[0] : (j == 1 ? w_pre[1] : nh.norm_weight[n]);
        rv = r_old + v;
        nh.residual[(int64_t)(m_base + m) * N + n] = rv;
        nh.a_out[(int64_t)(m_base + m) * N + n] = float_to_bf16_bits(rv * w_n);
      }
      sq[e] = rv * rv;
    } else if (live) {
      if (OUT_F32) reinterpret_cast<float*>(C)[(int64_t)(m_base + m) * ldc + n] = v;
      else reinterpret_cast<uint16_t*>(C)[(int64_t)(m_base + m) * ldc + n] = float_to_bf16_bits(v);
    }
  }
  if (nh.residual) {
    // row m's squares over this workgroup's columns, summed in a fixed order by one thread
    __syncthreads();
    for (int m = threadIdx.x; m < 16 * MB; m += blockDim.x) {
      float total = 0.f;
      for (int rb = 0; rb < (GATE_UP ? 1 : RB); ++rb)
        for (int q = 0; q < 4; ++q)
          for (int i = 0; i < 4; ++i) total += sq[(rb * MB + (m >> 4)) * 256 + 4 * ((m & 15) + 16 * q) + i];
      nh.ss_out[(int64_t)blockIdx.x * nh.ss_stride + m_base + m] = total;
    }
  }
}

// ---------------------------------------------------------------- residual add + RMS norm + product, fused
// For up to 16 rows:  r' = r + x   (x optional; r' is written to a second buffer, each workgroup a share of it)
//                     C  = ( rmsnorm(r') * w ) W^T
// The norm needs no pass of its own: the left operand is bf16(r' * w), the sum of squares of each row is
// gathered beside the products (every workgroup sees whole rows, its waves split K), and the row's
// rsqrt(mean + eps) scales the 32-bit result.  `rows` (optional) picks the rows of r and x.
template <int RB, bool GATE_UP>
__global__ __launch_bounds__(512) void norm_gemm_kernel(const float* __restrict__ R, const uint16_t* __restrict__ X,
                                                        float* __restrict__ R_out, const float* __restrict__ NW,
                                                        const int* __restrict__ rows, float eps,
                                                        const uint16_t* __restrict__ W, int64_t ldw,
                                                        uint16_t* __restrict__ C, int64_t ldc, int M, int N, int K) {
  extern __shared__ float red[];   // [waves][RB][256] sums, then [waves][16] squares
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = GATE_UP ? blockIdx.x * 16 : blockIdx.x * 16 * RB;
  const int steps = (K + 31) / 32;
  const int spw = (steps + nw - 1) / nw;
  const int s_begin = wave * spw;
  const int s_end = min(steps, s_begin + spw);
  float* red_ss = red + nw * RB * 256;

  f32x4 acc[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) acc[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
  const uint16_t* wrow[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    int row = GATE_UP ? n0 + (lane & 15) : n0 + 16 * rb + (lane & 15);
    row = row < N ? row : N - 1;
    if (GATE_UP && rb == 1) row += N;
    wrow[rb] = W + (int64_t)row * ldw;
  }
  const int m = lane & 15;
  const bool mok = m < M;
  const int64_t src = mok ? (rows ? rows[m] : m) : 0;
  const float* rrow = R + src * K;
  const uint16_t* xrow = X ? X + src * K : nullptr;
  float* orow = R_out ? R_out + (int64_t)(mok ? m : 0) * K : nullptr;
  float ss = 0.f;

  constexpr int CH = 4;
  for (int s0 = s_begin; s0 < s_end; s0 += CH) {
    bf16x8 w[CH][RB];
    f32x4 r0[CH], r1[CH], g0[CH], g1[CH];
    u32x4 xr[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int k = 32 * (s0 + c) + 8 * (lane >> 4);
      const bool kok = (s0 + c < s_end) && k < K;
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) w[c][rb] = kok ? W_LOAD(reinterpret_cast<const bf16x8*>(wrow[rb] + k)) : zero_bf16x8();
      const bool ok = kok && mok;
      r0[c] = ok ? *reinterpret_cast<const f32x4*>(rrow + k) : f32x4{0.f, 0.f, 0.f, 0.f};
      r1[c] = ok ? *reinterpret_cast<const f32x4*>(rrow + k + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
      xr[c] = (ok && xrow) ? *reinterpret_cast<const u32x4*>(xrow + k) : u32x4{0, 0, 0, 0};
      g0[c] = kok ? *reinterpret_cast<const f32x4*>(NW + k) : f32x4{0.f, 0.f, 0.f, 0.f};
      g1[c] = kok ? *reinterpret_cast<const f32x4*>(NW + k + 4) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      if (s0 + c >= s_end) break;
      const int k = 32 * (s0 + c) + 8 * (lane >> 4);
      float v[8] = {r0[c][0], r0[c][1], r0[c][2], r0[c][3], r1[c][0], r1[c][1], r1[c][2], r1[c][3]};
      const uint32_t xw[4] = {xr[c][0], xr[c][1], xr[c][2], xr[c][3]};
      const float gw[8] = {g0[c][0], g0[c][1], g0[c][2], g0[c][3], g1[c][0], g1[c][1], g1[c][2], g1[c][3]};
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        v[2 * i] += __uint_as_float(xw[i] << 16);
        v[2 * i + 1] += __uint_as_float(xw[i] & 0xffff0000u);
      }
      union {
        bf16x8 v8;
        uint16_t h[8];
      } a;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        ss += v[i] * v[i];
        a.h[i] = float_to_bf16_bits(v[i] * gw[i]);
      }
      // this workgroup's share of the new residual: the steps s with s % gridDim.x == blockIdx.x
      if (orow && mok && k < K && ((s0 + c) % gridDim.x) == blockIdx.x) {
        *reinterpret_cast<float4*>(orow + k) = float4{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<float4*>(orow + k + 4) = float4{v[4], v[5], v[6], v[7]};
      }
#pragma unroll
      for (int rb = 0; rb < RB; ++rb) acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[c][rb], a.v8, acc[rb], 0, 0, 0);
    }
  }
  // squares: the 4 lanes that share a row, then the waves
  ss += __shfl_xor(ss, 16, 64);
  ss += __shfl_xor(ss, 32, 64);
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) *reinterpret_cast<f32x4*>(red + ((wave * RB + rb) * 64 + lane) * 4) = acc[rb];
  if (lane < 16) red_ss[wave * 16 + lane] = ss;
  __syncthreads();
  constexpr int OB = GATE_UP ? 1 : RB;
  for (int e = threadIdx.x; e < OB * 256; e += blockDim.x) {
    const int blk = e >> 8, r = e & 255;
    const int ln = r >> 2, i = r & 3;
    const int mm = ln & 15;
    float v = 0.f, u = 0.f, sq = 0.f;
    for (int w = 0; w < nw; ++w) {
      v += red[(w * RB + blk) * 256 + r];
      if (GATE_UP) u += red[(w * RB + 1) * 256 + r];
      sq += red_ss[w * 16 + mm];
    }
    const float rstd = rsqrtf(sq / (float)K + eps);
    v *= rstd;
    if (GATE_UP) v = silu_f(v) * (u * rstd);
    const int n = n0 + 16 * blk + 4 * (ln >> 4) + i;
    if (n < N && mm < M) C[(int64_t)mm * ldc + n] = float_to_bf16_bits(v);
  }
}

// Compute units of the current device (256 on an MI355X); every count of workgroups or waves that is meant to fill
// the chip is derived from it.
static int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
  }
  return cus;
}

// Wave slots of the chip: 16 on each compute unit.
static int wave_slots() { return 16 * compute_units(); }

// R [*, K] float32 residual, X [*, K] bfloat16 or null, R_out [M, K] float32 or null (written when given),
// NW [K] float32 norm weight, rows [M] or null, W [N, K] (gate_up: [2 N, K]) bfloat16, C [M, N] bfloat16.
MI_EXPORT int mi_norm_gemm_skinny(int gate_up, const float* R, const void* X, float* R_out, const float* NW,
                                  const int* rows, float eps, const void* W, int64_t ldw, void* C, int64_t ldc, int M,
                                  int N, int K, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && M <= 16, "norm_gemm_skinny: M=%d; this kernel takes at most 16 rows", M);
  MI_REQUIRE(N > 0 && K > 0 && K % 8 == 0 && ldw % 8 == 0 && ldw >= K && ldc >= N, "norm_gemm_skinny: N=%d K=%d ldw=%lld",
             N, K, (long long)ldw);
  MI_REQUIRE(R && NW && W && C, "norm_gemm_skinny: missing operand");
  MI_REQUIRE(!(rows && R_out), "norm_gemm_skinny: a row selection cannot update the residual");
  if (M == 0) return 0;
  const int row_blocks = (N + 15) / 16;
  const int RB = gate_up ? 2 : (row_blocks >= 1024 ? 2 : 1);
  const int groups = gate_up ? row_blocks : (row_blocks + RB - 1) / RB;
  const int steps = (K + 31) / 32;
  int waves = (wave_slots() + groups - 1) / groups;
  if (waves > 8) waves = 8;
  if (waves > steps / 2) waves = steps / 2;
  if (waves < 1) waves = 1;
  const size_t lds = ((size_t)waves * RB * 256 + waves * 16) * sizeof(float);
  const dim3 grid(groups), block(64 * waves);
#define GO(rb, GU)                                                                                                  \
  norm_gemm_kernel<rb, GU><<<grid, block, lds, stream>>>(R, (const uint16_t*)X, R_out, NW, rows, eps,               \
                                                         (const uint16_t*)W, ldw, (uint16_t*)C, ldc, M, N, K)
  if (gate_up) GO(2, true);
  else if (RB == 2) GO(2, false);
  else GO(1, false);
#undef GO
  MI_CHECK_LAUNCH("norm_gemm_skinny");
  return 0;
}

// staging: 0 none, 1 the left operand's pieces, 2 both operands' (the mode for up to 16 rows)
static size_t skinny_lds_bytes(int waves, int RB, int MB, bool gate_up, int staging = 0, int M = 16) {
  const int OB = gate_up ? MB : RB * MB;
  const size_t sums = ((size_t)((waves + 1) / 2) * RB * MB * 256 + (size_t)OB * 256 + (size_t)waves * 64) * sizeof(float);
  const size_t stage = staging == 1   ? (size_t)waves * SKINNY_STAGE_KB(MB) * 1024
                       : staging == 2
                           ? (size_t)waves * (SKINNY_STAGE5_KB(RB) + (M * 4 * SKINNY_STAGE5_STEPS + 63) / 64) * 1024 +
                                 16 * 4 * SKINNY_STAGE5_STEPS * 16            // the last wave's reads of rows past M
                           : 0;
  return sums > stage ? sums : stage;
}

// Rows of W per workgroup and workgroups of the launch.  A matrix of few rows is cut finer than the 16 rows of a
// matrix-core tile when the left operand has at most 16 rows (with more, the operand's re-reads per workgroup
// would outweigh what the extra workgroups gain).
struct SkinnyGrid {
  int RB, rpg, groups;
};

static SkinnyGrid skinny_grid(bool gate_up, int N, int M) {
  const int row_blocks = (N + 15) / 16;
  const int cus = compute_units();
  SkinnyGrid g;
  g.rpg = 16;
  if (gate_up) {
    g.RB = 2;
    if (M <= 16) {
      const int rounds = (N + 16 * cus - 1) / (16 * cus);
      const int rpg = (N + cus * rounds - 1) / (cus * rounds);
      g.rpg = rpg < 4 ? 4 : (rpg > 16 ? 16 : rpg);
    }
    g.groups = (N + g.rpg - 1) / g.rpg;
  } else if (M <= 16 && row_blocks < 1024) {
    // A workgroup of 16 waves has a compute unit to itself, so the launch runs in rounds of as many workgroups as
    // there are units, and 320 workgroups take as long as 512.  The rows are shared out so that the last round is
    // as full as the others, up to 32 to a workgroup (two row blocks, which halves what the left operand's reads
    // add to the weights'): 1,024 rows on 256 units go as 256 groups of 4, 5,120 rows as 256 groups of 2 x 10,
    // 10,240 rows as 512 groups of 2 x 10.
    // (With fewer than 4 rows the left operand is a small part of the bytes, and the finer cut's extra workgroups
    // win: a row block each, then.)
    const int most = M < 4 ? 16 : 32;
    const int rounds = (N + most * cus - 1) / (most * cus);
    const int per_group = (N + cus * rounds - 1) / (cus * rounds);      // at most `most`
    if (per_group <= 16) {
      g.RB = 1;
      g.rpg = per_group < 4 ? 4 : per_group;
    } else {
      g.RB = 2;
      g.rpg = (per_group + 1) / 2;
    }
    g.groups = (N + g.rpg * g.RB - 1) / (g.rpg * g.RB);
  } else {
    g.RB = row_blocks >= 1024 ? 2 : 1;
    g.groups = (row_blocks + g.RB - 1) / g.RB;
  }
  return g;
}

// Waves per workgroup: enough to fill the chip (where one would do, four: a launch of thousands of workgroups then
// ends in smaller pieces; the output head takes 263 instead of 288 us); at least 2 steps of K per wave, at most 16.
static int skinny_waves(int groups, int steps, int RB, int MB, bool gate_up) {
  int waves = (wave_slots() + groups - 1) / groups;
  if (waves < 2) waves = 4;
  if (waves > 16) waves = 16;
  if (waves > steps / 2) waves = steps / 2;
  if (waves < 1) waves = 1;
  while (skinny_lds_bytes(waves, RB, MB, gate_up) > 64 * 1024 && waves > 1) waves /= 2;   // the default LDS allotment
  return waves;
}

constexpr size_t SKINNY_LDS_ROOM = 160 * 1024;      // what a workgroup may be given (launch_instance asks for it)

// The form that stages both operands keeps a wave's pieces of both in LDS: with two row blocks 16 waves' pieces are
// more than a compute unit has, and a few waves fewer still stream faster than 16 in another form (the 8B shape's
// [6144, 4096] at 16 rows: 14.9 -> 12.8 us; [5120, 8192] at 8 rows: 21.3 -> 18.5).  Returns 0 if even 8 do not fit.
// (Fewer waves cut k into other slices: the sums are then no longer those of the other forms bit for bit.)
static int both_staged_waves(int waves, int RB, int MB, bool gate_up, int M) {
  if (MB != 1) return 0;
  while (waves > 8 && skinny_lds_bytes(waves, RB, MB, gate_up, 2, M) > SKINNY_LDS_ROOM) --waves;
  return skinny_lds_bytes(waves, RB, MB, gate_up, 2, M) > SKINNY_LDS_ROOM ? 0 : waves;
}

template <int MB, int RB, bool F32, bool GU, int MODE>
static void launch_instance(dim3 grid, dim3 block, size_t lds, hipStream_t stream, const void* A, int64_t lda,
                            const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N, int K, int rpg,
                            const NormHalves& nh) {
  auto kernel = gemm_skinny_kernel<MB, RB, F32, GU, MODE>;
  if (MODE == 2 || MODE >= 4) {     // its staging pieces may need more than the default allotment of LDS
    static bool allowed = false;
    if (!allowed) {
      (void)hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      allowed = true;
    }
  }
  kernel<<<grid, block, lds, stream>>>((const uint16_t*)A, lda, (const uint16_t*)W, ldw, C, ldc, M, N, K, rpg, nh);
}

template <int MB, int RB>
static int launch(bool out_f32, bool gate_up, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                  int64_t ldc, int M_all, int N, int K, int waves, const SkinnyGrid& sg, const NormHalves& nh,
                  int want, int grid_y, hipStream_t stream) {
  // grid_y > 1: the rows of A are shared out too, 16 MB to a workgroup (the kernel takes its share of M_all)
  const dim3 grid(sg.groups, grid_y);
  const int M = grid_y > 1 ? 16 * MB : M_all;        // rows of A a workgroup stages
  const int64_t w_rows = gate_up ? 2 * (int64_t)N : N;
  const bool lean = K % 32 == 0 && w_rows * ldw * 2 < ((int64_t)1 << 32) && (int64_t)M_all * lda * 2 < ((int64_t)1 << 32) &&
                    (((uintptr_t)A | (uintptr_t)W) & 15) == 0;
  // want: the kernel's mode the caller asks for (1 .. 5); it is taken as far as the shape allows
  int mode = 0;
  if (lean) {
    mode = want < 1 ? 1 : want;
    const size_t room = SKINNY_LDS_ROOM;
    if (mode == 5) {
      const int nw = both_staged_waves(waves, RB, MB, gate_up, M);
      if (nw == 0) mode = 2;
      else waves = nw;
    }
    if ((mode == 3 || mode == 4) && K % 64 != 0) mode -= 2;
    if ((mode == 2 || mode == 4) && skinny_lds_bytes(waves, RB, MB, gate_up, 1) > room) mode -= 1;
  }
  const dim3 block(64 * waves);
  const size_t lds = skinny_lds_bytes(waves, RB, MB, gate_up, mode == 5 ? 2 : (mode == 2 || mode == 4) ? 1 : 0, M);
#define GO(F32, GU)                                                                                                  \
  {                                                                                                                  \
    if (mode == 5) {                                                                                                 \
      if constexpr (MB == 1)                                                                                         \
        launch_instance<MB, RB, F32, GU, 5>(grid, block, lds, stream, A, lda, W, ldw, C, ldc, M_all, N, K, sg.rpg, nh);  \
    } else if (mode == 4) launch_instance<MB, RB, F32, GU, 4>(grid, block, lds, stream, A, lda, W, ldw, C, ldc, M_all, N, K, sg.rpg, nh); \
    else if (mode == 3) launch_instance<MB, RB, F32, GU, 3>(grid, block, lds, stream, A, lda, W, ldw, C, ldc, M_all, N, K, sg.rpg, nh); \
    else if (mode == 2) launch_instance<MB, RB, F32, GU, 2>(grid, block, lds, stream, A, lda, W, ldw, C, ldc, M_all, N, K, sg.rpg, nh); \
    else if (mode == 1) launch_instance<MB, RB, F32, GU, 1>(grid, block, lds, stream, A, lda, W, ldw, C, ldc, M_all, N, K, sg.rpg, nh); \
    else launch_instance<MB, RB, F32, GU, 0>(grid, block, lds, stream, A, lda, W, ldw, C, ldc, M_all, N, K, sg.rpg, nh);  \
  }
  if (gate_up) {
    if constexpr (RB == 2) {
      if (out_f32) GO(true, true)
      else GO(false, true)
    }
  } else {
    if (out_f32) GO(true, false)
    else GO(false, false)
  }
#undef GO
  return 0;
}

// Waves per workgroup of the launch (variant as in mi_gemm_skinny_v, the kernel that owns whole rows; operands taken
// to be aligned): forms with the same number add the same products in the same order.
MI_EXPORT int mi_gemm_skinny_waves(int variant, int gate_up, int M, int N, int K) {
  if (M < 1 || M > 64 || N < 1 || K < 1) return 0;
  const SkinnyGrid sg = skinny_grid(gate_up != 0, N, M);
  const int MB = (M + 15) / 16;
  const int waves = skinny_waves(sg.groups, (K + 31) / 32, sg.RB, MB, gate_up != 0);
  if (variant == 5 && K % 32 == 0) {
    const int nw = both_staged_waves(waves, sg.RB, MB, gate_up != 0, M);
    if (nw) return nw;
  }
  return waves;
}

// Workgroups of the launch for M rows and an [N, K] matrix: `ss_out` holds that many rows of mi_gemm_skinny_ss_row(M).
MI_EXPORT int mi_gemm_skinny_groups(int gate_up, int N, int M) { return skinny_grid(gate_up != 0, N, M).groups; }
MI_EXPORT int mi_gemm_skinny_ss_row(int M) { return SS_ROW(M); }

// A [M, K], C [M, N] bfloat16 or float32; W [N, K], or with gate_up the fused matrix [2 N, K].
// Norm halves (see NormHalves; all optional): row_ss [ss_parts][ss_row(M)] and eps scale the rows of the result;
// residual [M, N] float32 + norm_weight [N] + a_out [M, N] bfloat16 + ss_out [groups][ss_row(M)] replace C.
static int skinny_rows(int out_f32, int gate_up, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                       int64_t ldc, int M, int N, int K, const float* row_ss, int ss_parts, float eps,
                       float* residual, const float* norm_weight, void* a_out, float* ss_out, int want,
                       hipStream_t stream) {
  MI_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: M=%d; this kernel takes at most 64 rows", M);
  MI_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: N=%d K=%d (K must be a multiple of 8)", N, K);
  MI_REQUIRE(lda % 8 == 0 && ldw % 8 == 0, "gemm_skinny: row strides (%lld, %lld) must be multiples of 8", (long long)lda,
             (long long)ldw);
  MI_REQUIRE(lda >= K && ldw >= K, "gemm_skinny: leading dimensions too small");
  MI_REQUIRE(residual || (C && ldc >= N), "gemm_skinny: no result buffer");
  MI_REQUIRE(!residual || (norm_weight && a_out && ss_out && !gate_up),
             "gemm_skinny: the residual form needs norm_weight, a_out and ss_out, and no gate|up");
  MI_REQUIRE(!row_ss || ss_parts > 0, "gemm_skinny: row_ss without parts");
  if (M == 0) return 0;
  const SkinnyGrid sg = skinny_grid(gate_up != 0, N, M);
  const int RB = sg.RB, groups = sg.groups;
  const int steps = (K + 31) / 32;
  const int MB = (M + 15) / 16;
  const int waves = skinny_waves(groups, steps, RB, MB, gate_up != 0);
  const NormHalves nh{row_ss, ss_parts, eps, residual, norm_weight, (uint16_t*)a_out, ss_out, SS_ROW(M)};
  if (want == 6 && M > 16) {
    // the rows of A shared out as well: blocks of 16 rows along the grid's second dimension, every workgroup the
    // kernel for up to 16 rows with both operands staged (or what of that the shape allows)
    const int gy = MB;
    const int w6 = skinny_waves(groups * gy, steps, RB, 1, gate_up != 0);
    if (RB == 1) launch<1, 1>(out_f32 != 0, gate_up != 0, A, lda, W, ldw, C, ldc, M, N, K, w6, sg, nh, 5, gy, stream);
    else launch<1, 2>(out_f32 != 0, gate_up != 0, A, lda, W, ldw, C, ldc, M, N, K, w6, sg, nh, 5, gy, stream);
    MI_CHECK_LAUNCH("gemm_skinny");
    return 0;
  }
  if (want == 6) want = 5;
#define CASE(mb, rb)                                                                                          \
  if (MB == mb && RB == rb) {                                                                                 \
    launch<mb, rb>(out_f32 != 0, gate_up != 0, A, lda, W, ldw, C, ldc, M, N, K, waves, sg, nh, want, 1, stream); \
    MI_CHECK_LAUNCH("gemm_skinny");                                                                           \
    return 0;                                                                                                 \
  }
  CASE(1, 1) CASE(2, 1) CASE(3, 1) CASE(4, 1) CASE(1, 2) CASE(2, 2) CASE(3, 2) CASE(4, 2)
#undef CASE
  MI_FAIL("gemm_skinny: no instance for M=%d", M);
}

MI_EXPORT int mi_gemm_skinny_ex(int out_f32, int gate_up, const void* A, int64_t lda, const void* W, int64_t ldw,
                                void* C, int64_t ldc, int M, int N, int K, const float* row_ss, int ss_parts,
                                float eps, float* residual, const float* norm_weight, void* a_out, float* ss_out,
                                hipStream_t stream) {
  return skinny_rows(out_f32, gate_up, A, lda, W, ldw, C, ldc, M, N, K, row_ss, ss_parts, eps, residual, norm_weight,
                     a_out, ss_out, 1, stream);
}

MI_EXPORT int mi_gemm_skinny(int out_f32, int gate_up, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                             int64_t ldc, int M, int N, int K, hipStream_t stream) {
  return mi_gemm_skinny_ex(out_f32, gate_up, A, lda, W, ldw, C, ldc, M, N, K, nullptr, 0, 0.f, nullptr, nullptr,
                           nullptr, nullptr, stream);
}

// ================================================================ the same product with k split across workgroups
// For more than 16 rows of A the kernel above pays for its left operand: every workgroup owns whole rows of the
// result, so it reads all of A, and what a compute unit draws from L2 between its weight loads is what the time
// grows with.  Here a workgroup owns SK_WN blocks of 16 weight rows and only a range of k: grid (row groups,
// splits).  The A columns of a chunk of SK_KC k's are read once per workgroup, coalesced, into LDS (two buffers: the
// next chunk's loads and the next chunk's weights are in flight while the current chunk is multiplied), every wave
// takes its operands from there, and a wave's weights come straight from global memory as above.  Each workgroup
// leaves a 32-bit partial result P[split][m][n]; a second kernel adds the partials of a result element in the
// order of the splits (so the sum does not depend on timing) and applies the same endings as the kernel above:
// row scale from partial sums of squares, gate|up activation, or residual add + next operand + sums of squares.
constexpr int SK_KC = 128;
constexpr int SK_STEPS = SK_KC / 32;
// LDS row stride in elements.  An operand read takes 16 bytes per lane from 16 rows, and the LDS serves lanes l .. l + 3
// and l + 16 .. l + 19 (the next 16 bytes of the same rows) together: 4 rows x 2 pieces fall into different banks when
// the stride is 8 (mod 16) banks of 4 bytes.
constexpr int SK_STRIDE = SK_KC + 16;
constexpr int SK_MAX_CHUNKS = 32;         // chunks of one split at most: columns per split <= 4096

// A wave owns RB blocks of 16 weight rows, a workgroup WN waves: 16 RB WN weight rows share every A chunk, and what
// a compute unit fetches beside its weights (the A columns, from L2) shrinks with that number: the time of this
// product follows the bytes a compute unit fetches, weights and A alike.
// D chunks are on their way at any time: chunk c + D (its A columns into staging registers, its weights into
// operand registers) is asked for when chunk c has been multiplied.  Loads come back in the order they were asked
// for, so the A columns of a chunk are asked for together with its weights, D chunks ahead, and waiting for them
// leaves the D - 1 later chunks in flight.
template <int MB, int WN, int RB, int D>
__global__ __launch_bounds__(64 * WN) void gemm_splitk_kernel(const uint16_t* __restrict__ A, int64_t lda,
                                                              const uint16_t* __restrict__ W, int64_t ldw,
                                                              float* __restrict__ P, int64_t ldp, void* __restrict__ C,
                                                              int64_t ldc, int out_f32, int M, int N, int K, int kr) {
  __shared__ __attribute__((aligned(16))) uint16_t a_lds[2][16 * MB * SK_STRIDE];
  constexpr int THREADS = 64 * WN;
  constexpr int ROWS_PER_PASS = THREADS / (SK_KC / 8);            // A rows that one load per thread covers
  constexpr int A_LOADS = (16 * MB + ROWS_PER_PASS - 1) / ROWS_PER_PASS;
  static_assert(THREADS % (SK_KC / 8) == 0, "a pass of the staging loads covers whole rows");
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int n0 = (blockIdx.x * WN + wave) * 16 * RB;
  const int split = blockIdx.y;
  const int k_lo = split * kr;
  const int k_hi = min(K, k_lo + kr);
  const int nchunks = k_hi > k_lo ? (k_hi - k_lo + SK_KC - 1) / SK_KC : 0;

  const uint16_t* wrow_base[RB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    int wr = n0 + 16 * rb + (lane & 15);
    wr = wr < N ? wr : N - 1;                   // rows past the end read the last row; they are never stored
    wrow_base[rb] = W + (int64_t)wr * ldw;
  }

  // this thread's pieces of an A chunk: 16 bytes of rows r0, r0 + ROWS_PER_PASS, ... at column 8 c16 of the chunk
  const int r0 = threadIdx.x / (SK_KC / 8), c16 = threadIdx.x % (SK_KC / 8);
  const int a_dst = r0 * SK_STRIDE + 8 * c16;

  f32x4 acc[RB][MB];
#pragma unroll
  for (int rb = 0; rb < RB; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};

  u32x4 a_st[D][A_LOADS];
  bf16x8 w[D][RB][SK_STEPS];
  // Loads are unconditional (a load inside a branch would end the straight-line code in which the compiler can
  // count the loads on their way): a piece outside the range reads a valid address instead and is zeroed afterwards.
  const int r_last = M - 1;
#define SK_FETCH(CH, SLOT)                                                                                    \
  {                                                                                                           \
    const int k0_ = k_lo + (CH) * SK_KC;                                                                      \
    const int ka = min(k0_ + 8 * c16, K - 8);                                                                 \
    _Pragma("unroll") for (int i = 0; i < A_LOADS; ++i) {                                                     \
      const int r = min(r0 + i * ROWS_PER_PASS, r_last);                                                      \
      a_st[SLOT][i] = *reinterpret_cast<const u32x4*>(A + (int64_t)r * lda + ka);                             \
    }                                                                                                         \
    _Pragma("unroll") for (int s = 0; s < SK_STEPS; ++s) {                                                    \
      const int k = min(k0_ + 32 * s + 8 * (lane >> 4), K - 8);                                               \
      _Pragma("unroll") for (int rb = 0; rb < RB; ++rb)                                                       \
        w[SLOT][rb][s] = W_LOAD(reinterpret_cast<const bf16x8*>(wrow_base[rb] + k));                          \
    }                                                                                                         \
  }
// zeroes what SK_FETCH read from outside the chunk's range (rows past M, columns past k_hi)
#define SK_MASK(CH, SLOT)                                                                                     \
  {                                                                                                           \
    const int k0_ = k_lo + (CH) * SK_KC;                                                                      \
    const bool col_ok = k0_ + 8 * c16 < k_hi;                                                                 \
    _Pragma("unroll") for (int i = 0; i < A_LOADS; ++i)                                                       \
      if (!(col_ok && r0 + i * ROWS_PER_PASS < M)) a_st[SLOT][i] = u32x4{0, 0, 0, 0};                         \
    _Pragma("unroll") for (int s = 0; s < SK_STEPS; ++s)                                                      \
      if (!(k0_ + 32 * s + 8 * (lane >> 4) < k_hi)) {                                                         \
        _Pragma("unroll") for (int rb = 0; rb < RB; ++rb) w[SLOT][rb][s] = zero_bf16x8();                     \
      }                                                                                                       \
  }
#pragma unroll
  for (int j = 0; j < D; ++j) SK_FETCH(j, j)      // chunks past the range read clamped addresses and are never used
  // The chunks are written out one after the other, with an exit after each: a loop would make the compiler wait
  // for all loads but the newest at its head (it cannot count loads in flight around a back edge), and the D chunks
  // on their way would shrink to one.  A split holds at most SK_MAX_CHUNKS chunks (the host cuts k accordingly).
#define SK_CHUNK(CI)                                                                                          \
  {                                                                                                           \
    constexpr int j = (CI) % D;                                                                               \
    uint16_t* buf = a_lds[(CI) & 1];                                                                          \
    SK_MASK(CI, j)                                                                                            \
    _Pragma("unroll") for (int i = 0; i < A_LOADS; ++i)                                                       \
      if (r0 + i * ROWS_PER_PASS < 16 * MB)                                                                   \
        *reinterpret_cast<u32x4*>(buf + a_dst + i * ROWS_PER_PASS * SK_STRIDE) = a_st[j][i];                  \
    __syncthreads(); /* the chunk is in LDS; every wave is past the chunk before last, whose buffer is next */ \
    _Pragma("unroll") for (int s = 0; s < SK_STEPS; ++s) {                                                    \
      _Pragma("unroll") for (int mb = 0; mb < MB; ++mb) {                                                     \
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(buf + (16 * mb + (lane & 15)) * SK_STRIDE + 32 * s + \
                                                          8 * (lane >> 4));                                   \
        _Pragma("unroll") for (int rb = 0; rb < RB; ++rb)                                                     \
          acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[j][rb][s], a, acc[rb][mb], 0, 0, 0);        \
      }                                                                                                       \
    }                                                                                                         \
    if ((CI) + D < SK_MAX_CHUNKS) SK_FETCH((CI) + D, j)                                                       \
    if (nchunks <= (CI) + 1) goto chunks_done;                                                                \
  }
  if (nchunks <= 0) goto chunks_done;
  SK_CHUNK(0) SK_CHUNK(1) SK_CHUNK(2) SK_CHUNK(3) SK_CHUNK(4) SK_CHUNK(5) SK_CHUNK(6) SK_CHUNK(7)
  SK_CHUNK(8) SK_CHUNK(9) SK_CHUNK(10) SK_CHUNK(11) SK_CHUNK(12) SK_CHUNK(13) SK_CHUNK(14) SK_CHUNK(15)
  SK_CHUNK(16) SK_CHUNK(17) SK_CHUNK(18) SK_CHUNK(19) SK_CHUNK(20) SK_CHUNK(21) SK_CHUNK(22) SK_CHUNK(23)
  SK_CHUNK(24) SK_CHUNK(25) SK_CHUNK(26) SK_CHUNK(27) SK_CHUNK(28) SK_CHUNK(29) SK_CHUNK(30) SK_CHUNK(31)
  static_assert(SK_MAX_CHUNKS == 32, "one SK_CHUNK per chunk of a split");
chunks_done:
#undef SK_CHUNK
#undef SK_MASK
#undef SK_FETCH
  // lane holds C^T[n0 + 16 rb + 4 (lane / 16) + i][16 mb + lane % 16]
#pragma unroll
  for (int rb = 0; rb < RB; ++rb) {
    if (n0 + 16 * rb >= N) break;   // a block past the last row (the row groups round N up) is not stored
    const int n = n0 + 16 * rb + 4 * (lane >> 4);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = 16 * mb + (lane & 15);
      if (m >= M) continue;
      if (C) {            // one split: the result itself
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) {
            if (out_f32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n + i] = acc[rb][mb][i];
            else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n + i] = float_to_bf16_bits(acc[rb][mb][i]);
          }
      } else {            // ldp covers whole blocks of 16 columns: columns past N are written and never read
        *reinterpret_cast<f32x4*>(P + ((int64_t)split * M + m) * ldp + n) = acc[rb][mb];
      }
    }
  }
}

// The same workgroup (128 weight rows, a range of k, partials P[split][m][n]) for matrices that are streamed from
// memory: both operands go straight to LDS (global_load_lds: lane i's 16 bytes land at base + 16 i) through a ring of
// SR_NBUF stages of 128 k, a wave's load instruction covering 1 KB (4 rows x 256 bytes) of whole memory lines, where
// the kernel above fetches the weights in the matrix cores' operand shape (16 rows x 64 bytes an instruction), which
// streams at two thirds of the rate.  Stage i + 2 is asked for before stage i is multiplied; a wave waits for its
// own loads of a stage by count (loads come back in the order they were asked for) and a barrier makes the stage
// every wave's.  A row's 16 pieces of 16 bytes are stored with their places exchanged by the row's number (piece q
// of row r at place q xor (r mod 16)), so that the 16 rows an operand read takes its pieces from lie in different
// banks.  k and every split's range are multiples of 128 here; rows of W past N and of A past M repeat the last row
// (loads to LDS cannot be replaced by zeros) and are never stored.
constexpr int SR_NBUF = 3;
constexpr int SR_WROWS = 128;
// END: how a workgroup leaves its sums.  0: partials P[split][m][n] for the kernel below (any number of splits).
// 1 (one split, nothing to do but store): the result itself.  2 (one split, a fused gate|up matrix of 2 N rows): the
// workgroup takes 64 gate rows and the 64 up rows of the same result columns, so a wave holds both sums of its
// columns and stores silu(gate) * up itself, the rows scaled first by rsqrt(sum_p row_ss[p][m] / K + eps) if row_ss
// is given (N is then the number of result columns).
struct RingEnd {
  const float* row_ss;      // [ss_parts][ss_row] or null
  int ss_parts;
  int ss_row;
  float eps;
};
template <int MB, int END>
__global__ __launch_bounds__(256) void gemm_splitk_ring_kernel(const uint16_t* __restrict__ A, int64_t lda,
                                                               const uint16_t* __restrict__ W, int64_t ldw,
                                                               float* __restrict__ P, int64_t ldp, void* __restrict__ C,
                                                               int64_t ldc, int out_f32, int M, int N, int K, int kr,
                                                               RingEnd e) {
  constexpr int AROWS = 16 * MB;
  constexpr int STAGE = (SR_WROWS + AROWS) * SK_KC;      // elements of a stage: the weight rows, then the rows of A
  constexpr int W_LOADS = SR_WROWS / 16;                 // wave loads (4 rows) of a stage that one of the 4 waves issues
  constexpr int LW = W_LOADS + MB;                       // with its loads of A
  constexpr int HALF = SR_WROWS / 2;
  extern __shared__ __attribute__((aligned(16))) uint16_t ring[];
  __shared__ float ss_part[4][64];                       // END 2 with row_ss: the four waves' shares of the rows' sums
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n0 = blockIdx.x * (END == 2 ? HALF : SR_WROWS);     // first weight row (END 2: first result column)
  const int split = blockIdx.y;
  const int k_lo = split * kr;
  const int k_hi = min(K, k_lo + kr);
  const int nst = k_hi > k_lo ? (k_hi - k_lo) / SK_KC : 0;
  // this lane's piece of every wave load: row rr of its 4 rows, place `at` of the row's 16
  const int rr = lane >> 4, at = lane & 15;
  const uint16_t* wsrc[W_LOADS];
  const uint16_t* asrc[MB];
#pragma unroll
  for (int j = 0; j < W_LOADS; ++j) {
    const int r = 4 * (wave + 4 * j) + rr;        // row of the stage
    int64_t wr;
    if (END == 2) wr = r < HALF ? min(n0 + r, N - 1) : N + min(n0 + r - HALF, N - 1);   // gate rows, then up rows
    else wr = min(n0 + r, N - 1);
    wsrc[j] = W + wr * ldw + k_lo + 8 * (at ^ (r & 15));
  }
#pragma unroll
  for (int j = 0; j < MB; ++j) {
    const int r = 4 * (wave + 4 * j) + rr;
    asrc[j] = A + (int64_t)min(r, M - 1) * lda + k_lo + 8 * (at ^ (r & 15));
  }
  // Every workgroup begins its walk over k somewhere else: side by side they would all ask for the same columns of
  // their rows, which lie a whole row apart in memory, that is (with rows of 8 KB, say) in the same few channels
  // (gate|up [24576, 4096] at 64 rows: 39.9 against 42.6 us; [32768, 4096]: 49.5 against 58.2).
  const int rot = nst > 0 ? (int)((((blockIdx.x + 1u) * 2654435761u + blockIdx.y * 40503u) >> 16) % (unsigned)nst) : 0;
  auto issue = [&](int st) {
    uint16_t* base = ring + (st % SR_NBUF) * STAGE;
    const int k0 = ((st + rot) % nst) * SK_KC;
#pragma unroll
    for (int j = 0; j < MB; ++j)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(asrc[j] + k0),
                                       (__attribute__((address_space(3))) void*)(base + SR_WROWS * SK_KC + (wave + 4 * j) * 512),
                                       16, 0, 0);
#pragma unroll
    for (int j = 0; j < W_LOADS; ++j)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(wsrc[j] + k0),
                                       (__attribute__((address_space(3))) void*)(base + (wave + 4 * j) * 512), 16, 0,
                                       W_LDS_AUX);
  };
  f32x4 acc[2][MB];
#pragma unroll
  for (int rb = 0; rb < 2; ++rb)
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) acc[rb][mb] = f32x4{0.f, 0.f, 0.f, 0.f};
  for (int st = 0; st < SR_NBUF - 1 && st < nst; ++st) issue(st);
  if (END == 2 && e.row_ss) {       // while the first stages are on their way: wave w adds parts w, w + 4, ... of row `lane`
    float ssum = 0.f;
    for (int p = wave; p < e.ss_parts; p += 4) ssum += e.row_ss[(int64_t)p * e.ss_row + min(lane, e.ss_row - 1)];
    ss_part[wave][lane] = ssum;     // read after the loop's barriers (a product has at least one stage)
  }
  const int row = lane & 15, kg = lane >> 4;
  // LDS rows of this wave's two blocks of 16 weight rows
  const int wrow0 = (END == 2 ? 16 * wave : 32 * wave) + row;
  const int wrow1 = (END == 2 ? HALF + 16 * wave : 32 * wave + 16) + row;
  for (int i = 0; i < nst; ++i) {
    // the compiler does not count the loads that write LDS: the waits are written out
    if (i + 1 < nst) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(LW) : "memory");     // stage i + 1 may still be on its way
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");   // stage i is here; everyone is past stage i - 1
    if (i + SR_NBUF - 1 < nst) issue(i + SR_NBUF - 1);                // into the buffer stage i - 1 was in
    const uint16_t* wst = ring + (i % SR_NBUF) * STAGE;
    const uint16_t* ast = wst + SR_WROWS * SK_KC;
#pragma unroll
    for (int s = 0; s < SK_STEPS; ++s) {
      const int place = 8 * ((4 * s + kg) ^ row);
      bf16x8 w[2];
      w[0] = *reinterpret_cast<const bf16x8*>(wst + wrow0 * SK_KC + place);
      w[1] = *reinterpret_cast<const bf16x8*>(wst + wrow1 * SK_KC + place);
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(ast + (16 * mb + row) * SK_KC + place);
#pragma unroll
        for (int rb = 0; rb < 2; ++rb)
          acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[rb], a, acc[rb][mb], 0, 0, 0);
      }
    }
  }
  if (END == 2) {
    // lane holds gate and up sums of result columns n0 + 16 wave + 4 (lane / 16) + i, row 16 mb + lane % 16
    const int nb = n0 + 16 * wave;
    if (nb >= N) return;
    const int n = nb + 4 * (lane >> 4);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = 16 * mb + (lane & 15);
      if (m >= M) continue;
      float rstd = 1.f;
      if (e.row_ss)
        rstd = rsqrtf(((ss_part[0][m] + ss_part[1][m]) + (ss_part[2][m] + ss_part[3][m])) / (float)K + e.eps);
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (n + i < N) {
          const float v = silu_f(acc[0][mb][i] * rstd) * (acc[1][mb][i] * rstd);
          if (out_f32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n + i] = v;
          else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n + i] = float_to_bf16_bits(v);
        }
    }
    return;
  }
  // lane holds C^T[n0 + 32 wave + 16 rb + 4 (lane / 16) + i][16 mb + lane % 16]
#pragma unroll
  for (int rb = 0; rb < 2; ++rb) {
    const int nb = n0 + 32 * wave + 16 * rb;
    if (nb >= N) break;
    const int n = nb + 4 * (lane >> 4);
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      const int m = 16 * mb + (lane & 15);
      if (m >= M) continue;
      if (END == 1) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < N) {
            if (out_f32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n + i] = acc[rb][mb][i];
            else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n + i] = float_to_bf16_bits(acc[rb][mb][i]);
          }
      } else {
        *reinterpret_cast<f32x4*>(P + ((int64_t)split * M + m) * ldp + n) = acc[rb][mb];
      }
    }
  }
}

// Adds the partials and finishes the product.  Grid (ceil(N / 256), ceil(M / waves)), 1 or 4 waves a workgroup (one
// where that still leaves few workgroups): wave w takes row waves * blockIdx.y + w, a lane 4 columns.  N counts result columns; with gate_up the partials hold 2 N (gate | up).
struct SplitkEnd {
  const float* row_ss;      // [ss_parts][ss_row]: scale row m by rsqrt(sum_p row_ss[p][m] / K + eps)
  int ss_parts;
  int ss_row;
  float eps;
  float* residual;          // [M, N]: residual += result; a_out = bf16(residual * norm_weight); ss_out[blockIdx.x][m]
  const float* norm_weight;
  uint16_t* a_out;
  float* ss_out;            // [gridDim.x][ss_row]
};

__global__ __launch_bounds__(256) void splitk_reduce_kernel(const float* __restrict__ P, int64_t ldp, int S,
                                                            void* __restrict__ C, int64_t ldc, int out_f32, int gate_up,
                                                            int M, int N, int K, SplitkEnd e) {
  const int lane = threadIdx.x & 63;
  const int m = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int n = blockIdx.x * 256 + 4 * lane;
  if (m >= M) return;                         // whole waves leave: no barrier below
  const bool live = n < N;                    // N is not a multiple of 4 in general: the last piece is partly live
  float ssum = 0.f;
  if (e.row_ss)
    for (int p = lane; p < e.ss_parts; p += 64) ssum += e.row_ss[(int64_t)p * e.ss_row + m];
  float r_old[4] = {0.f, 0.f, 0.f, 0.f}, nw[4] = {0.f, 0.f, 0.f, 0.f};
  if (e.residual && live) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (n + i < N) {
        r_old[i] = e.residual[(int64_t)m * N + n + i];
        nw[i] = e.norm_weight[n + i];
      }
  }
  f32x4 g = {0.f, 0.f, 0.f, 0.f}, u = {0.f, 0.f, 0.f, 0.f};
  if (live) {
    for (int s0 = 0; s0 < S; s0 += 8) {
      f32x4 pg[8], pu[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int s = s0 + j < S ? s0 + j : S - 1;        // a split again instead of a branch; it is not added
        const float* row = P + ((int64_t)s * M + m) * ldp;
        pg[j] = *reinterpret_cast<const f32x4*>(row + n);
        if (gate_up) pu[j] = *reinterpret_cast<const f32x4*>(row + N + n);    // N % 4 == 0 is required for gate|up
      }
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (s0 + j < S) {
          g += pg[j];
          if (gate_up) u += pu[j];
        }
    }
  }
  if (e.row_ss) {
    const float rstd = rsqrtf(wave_sum(ssum) / (float)K + e.eps);
    g *= rstd;
    u *= rstd;
  }
  float v[4] = {g[0], g[1], g[2], g[3]};
  if (gate_up) {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = silu_f(v[i]) * u[i];
  }
  if (e.residual) {
    float sq = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (live && n + i < N) {
        const float rv = r_old[i] + v[i];
        e.residual[(int64_t)m * N + n + i] = rv;
        e.a_out[(int64_t)m * N + n + i] = float_to_bf16_bits(rv * nw[i]);
        sq += rv * rv;
      }
    sq = wave_sum(sq);
    if (lane == 0) e.ss_out[(int64_t)blockIdx.x * e.ss_row + m] = sq;
    return;
  }
  if (!live) return;
#pragma unroll
  for (int i = 0; i < 4; ++i)
    if (n + i < N) {
      if (out_f32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n + i] = v[i];
      else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n + i] = float_to_bf16_bits(v[i]);
    }
}

// How a product of M rows with a [rows, K] matrix (rows = 2 N for gate|up) is cut: waves per workgroup (blocks of 16
// matrix rows), splits of k, columns per split, and the leading dimension of the partials.
struct SplitkPlan {
  int wn, rb, splits, kr, groups;
  int64_t ldp;
};

// for measurements: 0 keeps every k-split product on the kernel that fetches its weights into registers
static int g_splitk_ring = 1;
MI_EXPORT int mi_gemm_skinny_ring(int on) {
  const int was = g_splitk_ring;
  g_splitk_ring = on;
  return was;
}

static SplitkPlan splitk_plan(int M, int rows, int K, int want_splits) {
  SplitkPlan p;
  // weight rows per workgroup: 128 for matrices of many rows, 32 for those of few (which need the workgroups)
  const bool wide = rows >= 2048;
  p.wn = wide ? 4 : 2;
  p.rb = wide ? 2 : 1;
  const int tn = 16 * p.wn * p.rb;
  p.groups = (rows + tn - 1) / tn;
  // one workgroup for every compute unit: with twice as many (and half the k range each) every shape measured was
  // slower, by 5 to 25% (the ring kernel too: 64 rows of [4096, 12288] 27.4 us in 8 splits, 31 in 6 or 12, 39 in 2;
  // gate|up [24576, 4096] 46 us in its 192 row groups unsplit, 52 to 87 in 2 to 16 splits, whose partials grow)
  const int target = compute_units();
  int s = want_splits > 0 ? want_splits : (target + p.groups / 2) / p.groups;
  if (s < 1) s = 1;
  if (s > 32) s = 32;
  int kr = ((K + s - 1) / s + 31) / 32 * 32;
  if (K % SK_KC == 0) kr = (kr + SK_KC - 1) / SK_KC * SK_KC;      // whole stages of the ring kernel
  if (kr < 256) kr = 256;
  if (kr > SK_MAX_CHUNKS * SK_KC) kr = SK_MAX_CHUNKS * SK_KC;
  p.kr = kr;
  p.splits = (K + kr - 1) / kr;
  p.ldp = (int64_t)(rows + 15) / 16 * 16;
  return p;
}

// What a caller needs before a call of mi_gemm_skinny_v: rows of ss_out / row_ss that this product leaves when it
// is the first half of a norm (`ss_parts`), and the floats of scratch it needs (0 for every variant but 1).
MI_EXPORT int mi_gemm_skinny_plan(int variant, int gate_up, int M, int N, int K, int* ss_parts, int64_t* scratch_floats) {
  MI_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny_plan: M=%d N=%d K=%d", M, N, K);
  MI_REQUIRE(variant >= 0 && variant <= 6, "gemm_skinny_plan: variant %d", variant);
  if (variant != 1) {
    if (ss_parts) *ss_parts = skinny_grid(gate_up != 0, N, M).groups;
    if (scratch_floats) *scratch_floats = 0;
    return 0;
  }
  const SplitkPlan p = splitk_plan(M, gate_up ? 2 * N : N, K, 0);
  if (ss_parts) *ss_parts = (N + 255) / 256;
  if (scratch_floats) *scratch_floats = (int64_t)p.splits * M * p.ldp;
  return 0;
}

// mi_gemm_skinny_ex with a choice of kernel: variant 0 = every workgroup owns whole rows of the result (above),
// variant 1 = k split across workgroups, partial results in `scratch` (float, at least the plan's scratch_floats),
// added in the order of the splits by a second kernel that also does the endings; variant 2 = variant 0 with the left
// operand staged through LDS; variants 3 and 4 = variants 0 and 2 with the weights fetched in whole memory lines;
// variant 5 = both operands staged through LDS, for up to 16 rows (each where the shape allows it; else the nearest
// that it does); variant 6 = for more than 16 rows, the rows of A shared out across workgroups as well, 16 to each,
// every workgroup as in variant 5 (for up to 16 rows it is variant 5).  Variants 0, 2 and 5 add the same products in
// the same order: their results are equal bit for bit, and so are those of 3 and 4.
MI_EXPORT int mi_gemm_skinny_v(int variant, int out_f32, int gate_up, const void* A, int64_t lda, const void* W,
                               int64_t ldw, void* C, int64_t ldc, int M, int N, int K, const float* row_ss,
                               int ss_parts, float eps, float* residual, const float* norm_weight, void* a_out,
                               float* ss_out, float* scratch, int64_t scratch_floats, hipStream_t stream) {
  if (variant != 1 && variant >= 0 && variant <= 6)
    return skinny_rows(out_f32, gate_up, A, lda, W, ldw, C, ldc, M, N, K, row_ss, ss_parts, eps, residual, norm_weight,
                       a_out, ss_out, variant == 0 ? 1 : variant, stream);
  MI_REQUIRE(variant == 1, "gemm_skinny: variant %d", variant);
  MI_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: M=%d; this kernel takes at most 64 rows", M);
  MI_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: N=%d K=%d (K must be a multiple of 8)", N, K);
  MI_REQUIRE(lda % 8 == 0 && ldw % 8 == 0 && lda >= K && ldw >= K, "gemm_skinny: row strides (%lld, %lld)",
             (long long)lda, (long long)ldw);
  MI_REQUIRE(!gate_up || N % 4 == 0, "gemm_skinny: a gate|up product with k split needs a multiple of 4 columns, got %d",
             N);
  MI_REQUIRE(residual || (C && ldc >= N), "gemm_skinny: no result buffer");
  MI_REQUIRE(!residual || (norm_weight && a_out && ss_out && !gate_up),
             "gemm_skinny: the residual form needs norm_weight, a_out and ss_out, and no gate|up");
  MI_REQUIRE(!row_ss || ss_parts > 0, "gemm_skinny: row_ss without parts");
  if (M == 0) return 0;
  const int rows = gate_up ? 2 * N : N;
  const SplitkPlan p = splitk_plan(M, rows, K, 0);
  MI_REQUIRE(scratch && scratch_floats >= (int64_t)p.splits * M * p.ldp,
             "gemm_skinny: %lld floats of scratch, %lld are needed", (long long)scratch_floats,
             (long long)p.splits * M * p.ldp);
  const int MB = (M + 15) / 16;
  const dim3 grid(p.groups, p.splits);
  // matrices of many rows, k in whole stages, 16-byte alignment: the kernel that takes both operands through LDS
  if (g_splitk_ring && p.wn == 4 && K % SK_KC == 0 && p.kr % SK_KC == 0 && (((uintptr_t)A | (uintptr_t)W) & 15) == 0) {
    const size_t lds = (size_t)SR_NBUF * (SR_WROWS + 16 * MB) * SK_KC * sizeof(uint16_t);
    // one split: no partials.  A fused gate|up matrix is taken 64 gate and 64 up rows to a workgroup, which stores
    // the activation itself; a product with nothing to do at its end but store is stored by its workgroups.
    const int end = p.splits == 1 ? (gate_up ? 2 : (!row_ss && !residual ? 1 : 0)) : 0;
    const dim3 rgrid(end == 2 ? (N + SR_WROWS / 2 - 1) / (SR_WROWS / 2) : p.groups, p.splits);
    const RingEnd re{row_ss, ss_parts, SS_ROW(M), eps};
#define RING(mb, END)                                                                                            \
  {                                                                                                              \
    static bool allowed = false;                                                                                 \
    if (!allowed) {                                                                                              \
      /* what this instance needs, no more: its static LDS counts against the same 160 KB */                    \
      const hipError_t err_ = hipFuncSetAttribute((const void*)gemm_splitk_ring_kernel<mb, END>,                 \
                                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);         \
      MI_REQUIRE(err_ == hipSuccess, "gemm_skinny (k split, ring): %s", hipGetErrorString(err_));                \
      allowed = true;                                                                                            \
    }                                                                                                            \
    gemm_splitk_ring_kernel<mb, END><<<rgrid, 256, lds, stream>>>(                                               \
        (const uint16_t*)A, lda, (const uint16_t*)W, ldw, scratch, p.ldp, END ? C : nullptr, ldc, out_f32, M,     \
        END == 2 ? N : rows, K, p.kr, re);                                                                       \
  }
#define RING_MB(END)                                                                                             \
  if (MB == 1) RING(1, END) else if (MB == 2) RING(2, END) else if (MB == 3) RING(3, END) else RING(4, END)
    if (end == 2) { RING_MB(2) } else if (end == 1) { RING_MB(1) } else { RING_MB(0) }
#undef RING_MB
#undef RING
    MI_CHECK_LAUNCH("gemm_skinny (k split, ring)");
    if (end) return 0;
  } else {
#define GO(mb, wn, rb, d)                                                                                       \
  gemm_splitk_kernel<mb, wn, rb, d><<<grid, 64 * wn, 0, stream>>>((const uint16_t*)A, lda, (const uint16_t*)W,   \
                                                                  ldw, scratch, p.ldp, nullptr, ldc, out_f32, M, \
                                                                  rows, K, p.kr)
  if (p.wn == 4) {
    if (MB == 1) GO(1, 4, 2, 4);
    else if (MB == 2) GO(2, 4, 2, 3);
    else if (MB == 3) GO(3, 4, 2, 3);
    else GO(4, 4, 2, 3);
  } else {
    if (MB == 1) GO(1, 2, 1, 4);
    else if (MB == 2) GO(2, 2, 1, 4);
    else if (MB == 3) GO(3, 2, 1, 3);
    else GO(4, 2, 1, 3);
  }
#undef GO
  MI_CHECK_LAUNCH("gemm_skinny (k split)");
  }
  const SplitkEnd e{row_ss, ss_parts, SS_ROW(M), eps, residual, norm_weight, (uint16_t*)a_out, ss_out};
  const int red_waves = (int64_t)((N + 255) / 256) * M <= 2048 ? 1 : 4;
  splitk_reduce_kernel<<<dim3((N + 255) / 256, (M + red_waves - 1) / red_waves), 64 * red_waves, 0, stream>>>(
      scratch, p.ldp, p.splits, C, ldc, out_f32, gate_up, M, N, K, e);
  MI_CHECK_LAUNCH("gemm_skinny (k split, sum)");
  return 0;
}
