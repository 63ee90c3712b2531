// C[M, N] = A[M, K] * W[N, K]^T in bfloat16 for few rows of A (M <= 64): the decode step's projections
// and the output head, whose time is the time to stream W once from HBM.
//
// The product is computed transposed on the matrix cores, C^T[n, m] = W[n, :] . A[m, :], so that the
// 16 rows of an MFMA block are weight rows: each lane reads 16 contiguous bytes of a weight row straight
// from global memory into its operand slot (no LDS staging), and the few rows of A (which stay in L2)
// fill the other operand.  A workgroup owns 16 * RB weight rows; its waves split K and add their partial
// blocks through LDS.  32-bit accumulation; the result is stored as bfloat16 or float32.
//
// With SILU the left operand is made on the fly from a gate|up buffer [M, 2K]:
// a[m, k] = bf16( silu(gate[m, k]) * up[m, k] ), the feed-forward's activation
// (kernels/triton/silu_mul.py:33-37 of the reference) fused into the down projection.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ bf16x8 zero_bf16x8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.0f;
  return z;
}

__device__ __forceinline__ bf16x8 silu_mul8(const uint16_t* gate, const uint16_t* up) {
  const uint4 g = *reinterpret_cast<const uint4*>(gate);
  const uint4 u = *reinterpret_cast<const uint4*>(up);
  const uint32_t gw[4] = {g.x, g.y, g.z, g.w}, uw[4] = {u.x, u.y, u.z, u.w};
  union {
    bf16x8 v;
    uint16_t h[8];
  } r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    // hardware exp and reciprocal (about 1 ulp each): the result is rounded to bfloat16 anyway
    r.h[2 * i] = float_to_bf16_bits(g0 * __builtin_amdgcn_rcpf(1.f + __expf(-g0)) * u0);
    r.h[2 * i + 1] = float_to_bf16_bits(g1 * __builtin_amdgcn_rcpf(1.f + __expf(-g1)) * u1);
  }
  return r.v;
}

template <int MB, int RB, bool OUT_F32, bool SILU>
__global__ __launch_bounds__(1024) void gemm_skinny_kernel(const uint16_t* __restrict__ A, int64_t lda,
                                                           const uint16_t* __restrict__ W, int64_t ldw,
                                                           void* __restrict__ C, int64_t ldc, int M, int N, int K) {
  extern __shared__ float red[];   // [waves][RB * MB][256]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int nw = blockDim.x >> 6;
  const int n0 = blockIdx.x * 16 * RB;
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
    int row = n0 + 16 * rb + (lane & 15);
    row = row < N ? row : N - 1;            // rows past the end read the last row; they are never stored
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

#pragma unroll 4
  for (int s = s_begin; s < s_end; ++s) {
    const int k = 32 * s + 8 * (lane >> 4);
    const bool kok = k < K;                 // K is a multiple of 8: a lane's 8 elements are all in or all out
    bf16x8 w[RB], a[MB];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) w[rb] = kok ? *reinterpret_cast<const bf16x8*>(wrow[rb] + k) : zero_bf16x8();
#pragma unroll
    for (int mb = 0; mb < MB; ++mb) {
      if (kok && mok[mb]) {
        if (SILU) a[mb] = silu_mul8(arow[mb] + k, arow[mb] + K + k);
        else a[mb] = *reinterpret_cast<const bf16x8*>(arow[mb] + k);
      } else {
        a[mb] = zero_bf16x8();
      }
    }
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        acc[rb][mb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[rb], a[mb], acc[rb][mb], 0, 0, 0);
  }

  // lane holds C^T[n0 + 16 rb + 4 (lane / 16) + i][16 mb + lane % 16]
  if (nw > 1) {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb)
        *reinterpret_cast<f32x4*>(red + ((wave * RB * MB + rb * MB + mb) * 64 + lane) * 4) = acc[rb][mb];
    __syncthreads();
    // element e of the workgroup's result: block e / 256, lane (e % 256) / 4, register e % 4
    for (int e = threadIdx.x; e < RB * MB * 256; e += blockDim.x) {
      const int blk = e >> 8, r = e & 255;
      float v = 0.f;
      for (int w = 0; w < nw; ++w) v += red[(w * RB * MB + blk) * 256 + r];
      const int ln = r >> 2, i = r & 3;
      const int n = n0 + 16 * (blk / MB) + 4 * (ln >> 4) + i;
      const int m = 16 * (blk % MB) + (ln & 15);
      if (n < N && m < M) {
        if (OUT_F32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n] = v;
        else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n] = float_to_bf16_bits(v);
      }
    }
  } else {
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
      for (int mb = 0; mb < MB; ++mb) {
        const int m = 16 * mb + (lane & 15);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int n = n0 + 16 * rb + 4 * (lane >> 4) + i;
          if (n < N && m < M) {
            if (OUT_F32) reinterpret_cast<float*>(C)[(int64_t)m * ldc + n] = acc[rb][mb][i];
            else reinterpret_cast<uint16_t*>(C)[(int64_t)m * ldc + n] = float_to_bf16_bits(acc[rb][mb][i]);
          }
        }
      }
  }
}

template <int MB, int RB>
static int launch(bool out_f32, bool silu, const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc,
                  int M, int N, int K, int waves, hipStream_t stream) {
  const dim3 grid((N + 16 * RB - 1) / (16 * RB));
  const dim3 block(64 * waves);
  const size_t lds = waves > 1 ? (size_t)waves * RB * MB * 256 * sizeof(float) : 0;
#define GO(F32, SILU)                                                                                              \
  gemm_skinny_kernel<MB, RB, F32, SILU><<<grid, block, lds, stream>>>((const uint16_t*)A, lda, (const uint16_t*)W, \
                                                                      ldw, C, ldc, M, N, K)
  if (out_f32 && silu) GO(true, true);
  else if (out_f32) GO(true, false);
  else if (silu) GO(false, true);
  else GO(false, false);
#undef GO
  return 0;
}

// A [M, K] (or, with silu, the gate|up buffer [M, 2K]), W [N, K], C [M, N] bfloat16 or float32.
MI_EXPORT int mi_gemm_skinny(int out_f32, int silu, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                             int64_t ldc, int M, int N, int K, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && M <= 64, "gemm_skinny: M=%d; this kernel takes at most 64 rows", M);
  MI_REQUIRE(N > 0 && K > 0 && K % 8 == 0, "gemm_skinny: N=%d K=%d (K must be a multiple of 8)", N, K);
  MI_REQUIRE(lda % 8 == 0 && ldw % 8 == 0, "gemm_skinny: row strides (%lld, %lld) must be multiples of 8", (long long)lda,
             (long long)ldw);
  MI_REQUIRE(lda >= (silu ? 2 * (int64_t)K : K) && ldw >= K && ldc >= N, "gemm_skinny: leading dimensions too small");
  if (M == 0) return 0;
  const int row_blocks = (N + 15) / 16;
  const int RB = row_blocks >= 1024 ? 2 : 1;
  const int groups = (row_blocks + RB - 1) / RB;
  const int steps = (K + 31) / 32;
  // enough waves to fill the chip, at least 2 steps of K per wave, at most 16 waves per workgroup
  int waves = (4096 + groups - 1) / groups;
  if (waves > 16) waves = 16;
  if (waves > steps / 2) waves = steps / 2;
  if (waves < 1) waves = 1;
  const int MB = (M + 15) / 16;
  size_t lds = waves > 1 ? (size_t)waves * RB * MB * 1024 : 0;
  while (lds > 64 * 1024 && waves > 1) {     // the default LDS allotment of a workgroup
    waves /= 2;
    lds = waves > 1 ? (size_t)waves * RB * MB * 1024 : 0;
  }
#define CASE(mb, rb)                                                                                          \
  if (MB == mb && RB == rb) {                                                                                 \
    launch<mb, rb>(out_f32 != 0, silu != 0, A, lda, W, ldw, C, ldc, M, N, K, waves, stream);                \
    MI_CHECK_LAUNCH("gemm_skinny");                                                                           \
    return 0;                                                                                                 \
  }
  CASE(1, 1) CASE(2, 1) CASE(3, 1) CASE(4, 1) CASE(1, 2) CASE(2, 2) CASE(3, 2) CASE(4, 2)
#undef CASE
  MI_FAIL("gemm_skinny: no instance for M=%d", M);
}
