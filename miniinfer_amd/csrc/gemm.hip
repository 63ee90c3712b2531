// C[M, N] = A[M, K] * W[N, K]^T  (x @ W^T, the linear layer of miniinfer/layers/linear.py:4-33)
// with 32-bit FMA accumulation and no reduced-precision matrix instruction: this is the matrix
// product of the true 32-bit path, and the any-shape fallback of the bfloat16 path.
// The sum over K runs in one fixed order for every output element, whatever M is, so a row's
// result does not depend on what else is in the batch.
#include "common.h"

#define BM 64
#define BN 64
#define BK 16

template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const TA* __restrict__ A, int64_t lda,
                                                      const TA* __restrict__ W, int64_t ldw, TC* __restrict__ C,
                                                      int64_t ldc, int M, int N, int K) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15;   // 4 columns each
  const int ty = tid >> 4;   // 4 rows each
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  const int lr = tid >> 2;        // 0..63: tile row this thread loads
  const int lk = (tid & 3) * 4;   // 0,4,8,12: first k it loads

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    {
      const int m = m0 + lr;
      const int n = n0 + lr;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int k = k0 + lk + j;
        As[lk + j][lr] = (m < M && k < K) ? to_float(A[(int64_t)m * lda + k]) : 0.f;
        Ws[lk + j][lr] = (n < N && k < K) ? to_float(W[(int64_t)n * ldw + k]) : 0.f;
      }
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(int64_t)m * ldc + n] = from_float<TC>(acc[i][j]);
    }
  }
}

// The same product for up to 16 rows of A (a decode step of the 32-bit path), where the 64 x 64 tiles above would
// leave the chip idle: a workgroup takes 16 rows of W and all rows of A, one result element per thread, chunks of
// 64 k through LDS with the next chunk's loads in flight.  Every element is summed over k in the same order, with
// the same fused multiply-adds, as in the kernel above: a row's result is bit for bit what it is there.
#define FK 64
template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_few_rows_kernel(const TA* __restrict__ A, int64_t lda,
                                                               const TA* __restrict__ W, int64_t ldw,
                                                               TC* __restrict__ C, int64_t ldc, int M, int N, int K) {
  __shared__ float As[16][FK + 1];
  __shared__ float Ws[16][FK + 1];
  const int tid = threadIdx.x;
  const int m = tid >> 4;          // the thread's row of A (and the row of A it loads)
  const int nl = tid & 15;         // its row of W within the workgroup's 16
  const int n0 = blockIdx.x * 16;
  const int lk = (tid & 15) * 4;   // first k of the chunk that it loads: rows tid / 16 of A and of W
  const bool a_ok = m < M, w_ok = n0 + m < N;
  const TA* arow = A + (int64_t)(a_ok ? m : 0) * lda;
  const TA* wrow = W + (int64_t)(w_ok ? n0 + m : 0) * ldw;
  float ar[4], wr[4];
#define FEW_FETCH(K0)                                                                          \
  _Pragma("unroll") for (int j = 0; j < 4; ++j) {                                              \
    const int k = (K0) + lk + j;                                                               \
    ar[j] = (a_ok && k < K) ? to_float(arow[k]) : 0.f;                                         \
    wr[j] = (w_ok && k < K) ? to_float(wrow[k]) : 0.f;                                         \
  }
  FEW_FETCH(0)
  float acc = 0.f;
  for (int k0 = 0; k0 < K; k0 += FK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      As[m][lk + j] = ar[j];
      Ws[m][lk + j] = wr[j];
    }
    __syncthreads();
    if (k0 + FK < K) FEW_FETCH(k0 + FK)
#pragma unroll
    for (int kk = 0; kk < FK; ++kk) acc = fmaf(As[m][kk], Ws[nl][kk], acc);
    __syncthreads();
  }
#undef FEW_FETCH
  if (m < M && n0 + nl < N) C[(int64_t)m * ldc + n0 + nl] = from_float<TC>(acc);
}

// in_dtype: dtype of A and W; out_dtype: dtype of C.
MI_EXPORT int mi_gemm_nt(int in_dtype, int out_dtype, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                         int64_t ldc, int M, int N, int K, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_nt: bad sizes M=%d N=%d K=%d", M, N, K);
  MI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_nt: leading dimensions (%lld, %lld, %lld) too small for K=%d N=%d",
             (long long)lda, (long long)ldw, (long long)ldc, K, N);
  if (M == 0) return 0;
  const bool few = M <= 16;
  dim3 grid(few ? ceil_div(N, 16) : ceil_div(N, BN), few ? 1 : ceil_div(M, BM));
  MI_REQUIRE(grid.y <= 65535, "gemm_nt: M=%d too large for one launch", M);
#define LAUNCH(TA, TC)                                                                                              \
  if (few)                                                                                                          \
    gemm_nt_few_rows_kernel<TA, TC><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TA*)W, ldw, (TC*)C, ldc, M, \
                                                              N, K);                                               \
  else                                                                                                              \
    gemm_nt_kernel<TA, TC><<<grid, 256, 0, stream>>>((const TA*)A, lda, (const TA*)W, ldw, (TC*)C, ldc, M, N, K)
  if (in_dtype == MI_DTYPE_F32 && out_dtype == MI_DTYPE_F32) {
    LAUNCH(float, float);
  } else if (in_dtype == MI_DTYPE_BF16 && out_dtype == MI_DTYPE_BF16) {
    LAUNCH(bf16, bf16);
  } else if (in_dtype == MI_DTYPE_BF16 && out_dtype == MI_DTYPE_F32) {
    LAUNCH(bf16, float);
  } else {
    MI_FAIL("gemm_nt: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
  }
#undef LAUNCH
  MI_CHECK_LAUNCH("gemm_nt");
  return 0;
}
