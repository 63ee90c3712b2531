// C[M, N] = A[M, K] * W[N, K]^T in bfloat16 for few rows of A (M <= 64): the decode step's projections
// and the output head, whose time is the time to stream W once from HBM.
//
// The product is computed transposed on the matrix cores, C^T[n, m] = W[n, :] . A[m, :], so that the
// 16 rows of an MFMA block are weight rows: each lane reads 16 contiguous bytes of a weight row straight
// from global memory into its operand slot (no LDS staging), and the few rows of A (which stay in L2)
// fill the other operand.  A workgroup owns 16 * RB weight rows; its waves split K and add their partial
// blocks through LDS.  32-bit accumulation; the result is stored as bfloat16 or float32.
//
// With GATE_UP, W is a fused gate|up matrix [2 N, K] (gate rows first) and the result is the feed-forward's
// activation C[m, n] = silu(A W_gate^T)[m, n] * (A W_up^T)[m, n] (kernels/triton/silu_mul.py:33-37 of the
// reference), made from the 32-bit sums of gate row n and up row n, which the same workgroup owns.
#include "common.h"

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
struct NormHalves {
  const float* row_ss;      // [ss_parts][SS_ROW(M)]
  int ss_parts;
  float eps;
  float* residual;          // [M, N] float32, leading dimension N
  const float* norm_weight; // [N]
  uint16_t* a_out;          // [M, N] bfloat16, leading dimension N
  float* ss_out;            // [gridDim.x][SS_ROW(M)]
};

template <int MB, int RB, bool OUT_F32, bool GATE_UP>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(const uint16_t* __restrict__ A, int64_t lda,
                                                           const uint16_t* __restrict__ W, int64_t ldw,
                                                           void* __restrict__ C, int64_t ldc, int M, int N, int K,
                                                           int rpg, NormHalves nh) {
  extern __shared__ float red[];   // [(waves + 1) / 2][RB * MB][256], then (norm halves) [OB * 256] squares, [waves][64] sums
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  // GATE_UP: RB == 2, row block 0 = gate rows n0.., row block 1 = up rows N + n0..; N counts output columns
  // rpg: rows of W per workgroup and row block when RB == 1 or GATE_UP: 16, or fewer so that the workgroups fill
  // whole rounds of the compute units (the lanes of the other rows then load nothing and their results are dropped)
  constexpr bool CUT = GATE_UP || RB == 1;
  const int n0 = CUT ? blockIdx.x * rpg : blockIdx.x * 16 * RB;
  const int n_end = min(N, n0 + (CUT ? rpg : 16 * RB));
  const bool w_live = !CUT || (lane & 15) < rpg;
  const int steps = (K + 31) / 32;
  const int spw = (steps + nw - 1) / nw;
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
    int row = GATE_UP ? n0 + (lane & 15) : n0 + 16 * rb + (lane & 15);
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

  // What the norm halves read is asked for before the weights, so that the end of the kernel does not wait for
  // memory again: the partial sums of squares of row (thread % SS), parts (thread / SS), + threads / SS, ...; and
  // the residual and norm weight of the first two result elements this thread will finish.
  constexpr int OBLK = GATE_UP ? MB : RB * MB;
  constexpr int SS = SS_ROW(16 * MB);
  float my_ss = 0.f;
  if (nh.row_ss) {
    const int m = threadIdx.x % SS;
    for (int p = threadIdx.x / SS; p < nh.ss_parts; p += blockDim.x / SS) my_ss += nh.row_ss[(int64_t)p * SS + m];
  }
  float r_pre[2] = {0.f, 0.f}, w_pre[2] = {0.f, 0.f};
  if (nh.residual) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int e = threadIdx.x + j * blockDim.x;
      const int blk = e >> 8, ln = (e & 255) >> 2, i = e & 3;
      const int n = n0 + 16 * (blk / MB) + 4 * (ln >> 4) + i;
      const int m = 16 * (blk % MB) + (ln & 15);
      if (e < OBLK * 256 && n < n_end && m < M) {
        r_pre[j] = nh.residual[(int64_t)m * N + n];
        w_pre[j] = nh.norm_weight[n];
      }
    }
  }

  // Steps are taken CH at a time: first every load of the chunk is issued (weights, and the raw left operand),
  // then the operands are converted and multiplied, so one memory round trip covers CH steps.
  constexpr int CH = MB == 1 ? 8 : (MB == 2 ? 4 : 2);   // what fits the 128 registers of a 16-wave workgroup
  for (int s0 = s_begin; s0 < s_end; s0 += CH) {
    bf16x8 w[CH][RB];
    u32x4 ar[CH][MB];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int k = 32 * (s0 + c) + 8 * (lane >> 4);
      const bool kok = (s0 + c < s_end) && k < K;   // K is a multiple of 8: a lane's 8 elements are all in or all out
#pragma unroll
      for (int rb = 0; rb < RB; ++rb)
        w[c][rb] = (kok && w_live) ? *reinterpret_cast<const bf16x8*>(wrow[rb] + k) : zero_bf16x8();
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
    const int n = n0 + 16 * (GATE_UP ? 0 : blk / MB) + 4 * (ln >> 4) + i;
    const int m = 16 * (blk % MB) + (ln & 15);
    if (nh.row_ss) {
      float total = 0.f;
      for (int w = 0; w < nw; ++w) total += ss_part[w * 64 + m];
      const float rstd = rsqrtf(total / (float)K + nh.eps);
      v *= rstd;
      u *= rstd;
    }
    if (GATE_UP) v = silu_f(v) * u;
    const bool live = n < n_end && m < M;
    if (nh.residual) {
      float rv = 0.f;
      if (live) {
        const int j = (e - (int)threadIdx.x) / (int)blockDim.x;
        const float r_old = j == 0 ? r_pre[0] : (j == 1 ? r_pre[1] : nh.residual[(int64_t)m * N + n]);
        const float w_n = j == 0 ? w_pre[0] : (j == 1 ? w_pre[1] : nh.norm_weight[n]);
        rv = r_old + v;
        nh.residual[(int64_t)m * N + n] = rv;
        nh.a_out[(int64_t)m * N + n] = float_to_bf16_bits(rv * w_n);
      }
      sq[e] = rv * rv;
    } else if (live) {
      if (OUT_F32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n] = v;
      else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n] = float_to_bf16_bits(v);
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
      nh.ss_out[(int64_t)blockIdx.x * SS + m] = total;
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
      for (int rb = 0; rb < RB; ++rb) w[c][rb] = kok ? *reinterpret_cast<const bf16x8*>(wrow[rb] + k) : zero_bf16x8();
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
  int waves = (4096 + groups - 1) / groups;
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

static size_t skinny_lds_bytes(int waves, int RB, int MB, bool gate_up) {
  const int OB = gate_up ? MB : RB * MB;
  return ((size_t)((waves + 1) / 2) * RB * MB * 256 + (size_t)OB * 256 + (size_t)waves * 64) * sizeof(float);
}

// Rows of W per workgroup and workgroups of the launch.  A matrix of few rows is cut finer than the 16 rows of a
// matrix-core tile when the left operand has at most 16 rows (with more, the operand's re-reads per workgroup
// would outweigh what the extra workgroups gain).
struct SkinnyGrid {
  int RB, rpg, groups;
};

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

static SkinnyGrid skinny_grid(bool gate_up, int N, int M) {
  const int row_blocks = (N + 15) / 16;
  SkinnyGrid g;
  g.RB = gate_up ? 2 : (row_blocks >= 1024 ? 2 : 1);
  g.rpg = 16;
  if ((gate_up || g.RB == 1) && M <= 16) {
    // A workgroup of 16 waves has a compute unit to itself, so the launch runs in rounds of as many workgroups as
    // there are units, and 320 workgroups take as long as 512.  The rows are shared out so that the last round is
    // as full as the others: 5,120 rows on 256 units go as 512 groups of 10, 1,024 rows as 256 groups of 4.
    const int cus = compute_units();
    const int rounds = (N + 16 * cus - 1) / (16 * cus);
    const int rpg = (N + cus * rounds - 1) / (cus * rounds);
    g.rpg = rpg < 4 ? 4 : (rpg > 16 ? 16 : rpg);
  }
  g.groups = (gate_up || g.RB == 1) ? (N + g.rpg - 1) / g.rpg : (row_blocks + g.RB - 1) / g.RB;
  return g;
}

template <int MB, int RB>
static int launch(bool out_f32, bool gate_up, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                  int64_t ldc, int M, int N, int K, int waves, const SkinnyGrid& sg, const NormHalves& nh,
                  hipStream_t stream) {
  const dim3 grid(sg.groups);
  const dim3 block(64 * waves);
  const size_t lds = skinny_lds_bytes(waves, RB, MB, gate_up);
#define GO(F32, GU)                                                                                              \
  gemm_skinny_kernel<MB, RB, F32, GU><<<grid, block, lds, stream>>>((const uint16_t*)A, lda, (const uint16_t*)W, \
                                                                    ldw, C, ldc, M, N, K, sg.rpg, nh)
  if (gate_up) {
    if constexpr (RB == 2) {
      if (out_f32) GO(true, true);
      else GO(false, true);
    }
  } else {
    if (out_f32) GO(true, false);
    else GO(false, false);
  }
#undef GO
  return 0;
}

// Workgroups of the launch for M rows and an [N, K] matrix: `ss_out` holds that many rows of mi_gemm_skinny_ss_row(M).
MI_EXPORT int mi_gemm_skinny_groups(int gate_up, int N, int M) { return skinny_grid(gate_up != 0, N, M).groups; }
MI_EXPORT int mi_gemm_skinny_ss_row(int M) { return SS_ROW(M); }

// A [M, K], C [M, N] bfloat16 or float32; W [N, K], or with gate_up the fused matrix [2 N, K].
// Norm halves (see NormHalves; all optional): row_ss [ss_parts][ss_row(M)] and eps scale the rows of the result;
// residual [M, N] float32 + norm_weight [N] + a_out [M, N] bfloat16 + ss_out [groups][ss_row(M)] replace C.
MI_EXPORT int mi_gemm_skinny_ex(int out_f32, int gate_up, const void* A, int64_t lda, const void* W, int64_t ldw,
                                void* C, int64_t ldc, int M, int N, int K, const float* row_ss, int ss_parts,
                                float eps, float* residual, const float* norm_weight, void* a_out, float* ss_out,
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
  // enough waves to fill the chip (where one would do, four: a launch of thousands of workgroups then ends in
  // smaller pieces; the output head takes 263 instead of 288 us); at least 2 steps of K per wave, at most 16 waves
  // per workgroup
  int waves = (4096 + groups - 1) / groups;
  if (waves < 2) waves = 4;
  if (waves > 16) waves = 16;
  if (waves > steps / 2) waves = steps / 2;
  if (waves < 1) waves = 1;
  const int MB = (M + 15) / 16;
  while (skinny_lds_bytes(waves, RB, MB, gate_up != 0) > 64 * 1024 && waves > 1) waves /= 2;   // the default LDS allotment
  const NormHalves nh{row_ss, ss_parts, eps, residual, norm_weight, (uint16_t*)a_out, ss_out};
#define CASE(mb, rb)                                                                                          \
  if (MB == mb && RB == rb) {                                                                                 \
    launch<mb, rb>(out_f32 != 0, gate_up != 0, A, lda, W, ldw, C, ldc, M, N, K, waves, sg, nh, stream);          \
    MI_CHECK_LAUNCH("gemm_skinny");                                                                           \
    return 0;                                                                                                 \
  }
  CASE(1, 1) CASE(2, 1) CASE(3, 1) CASE(4, 1) CASE(1, 2) CASE(2, 2) CASE(3, 2) CASE(4, 2)
#undef CASE
  MI_FAIL("gemm_skinny: no instance for M=%d", M);
}

MI_EXPORT int mi_gemm_skinny(int out_f32, int gate_up, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                             int64_t ldc, int M, int N, int K, hipStream_t stream) {
  return mi_gemm_skinny_ex(out_f32, gate_up, A, lda, W, ldw, C, ldc, M, N, K, nullptr, 0, 0.f, nullptr, nullptr,
                           nullptr, nullptr, stream);
}
