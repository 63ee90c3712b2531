// C[M, N] = A[M, K] * W[N, K]^T  (x @ W^T, the linear layer of miniinfer/layers/linear.py:4-33)
// with 32-bit FMA accumulation and no reduced-precision matrix instruction: this is the matrix
// product of the true 32-bit path, and the any-shape fallback of the bfloat16 path.
//
// One order of summation for every result element, whatever M is and whichever kernel runs it: k is cut into
// chunks of 64; a chunk's products are added by one chain of fused multiply-adds, k ascending, from zero; the
// chunks' sums are added one after the other, first chunk first.  So a row's result does not depend on what else
// is in the batch, bit for bit, and the chunks are what the kernel for few rows works on side by side.
#include "common.h"
#include <type_traits>

#define BM 64
#define BN 64
#define BK 16
#define CHUNK_K 64        // k per chunk of the order of summation (a multiple of BK)

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

  float acc[4][4], tot[4][4];     // the running chunk's chain, and the sum of the chunks before it
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = tot[i][j] = 0.f;

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
    if ((k0 + BK) % CHUNK_K == 0 || k0 + BK >= K) {      // a chunk ends here
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          tot[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
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
      if (n < N) C[(int64_t)m * ldc + n] = from_float<TC>(tot[i][j]);
    }
  }
}

// The same product for up to 16 rows of A (a decode step of the 32-bit path), where the time is the time to stream
// W and the 64 x 64 tiles above would leave most of the chip idle.  A workgroup owns R rows of W (4, 8 or 16) and has
// R x SCH threads: thread (r, c) takes chunk c of a block
// of SCH chunks of row r, fetches its 64 weights itself (16 loads of 16 bytes, all on their way at once, no branch
// between them), and multiplies them with that chunk of every row of A, which the workgroup has staged in LDS once
// per block (a chunk's 64 values every 68 floats, so that the chunks' reads fall into different banks).  A thread's
// MT chains (one per row of A) are the order of summation's chunk chains; the chunks' sums go through LDS to one
// thread per result element, which adds them in order.  MT = 4, 8 or 16 rows of A are held; SCH = 16, 32 or 48 chunks
// (1,024 to 3,072 k) a block, as many as k has where the staged rows fit LDS; VEC: k, the row strides and the bases allow 16-byte
// accesses (else one element at a time).
#define SPAD 68           // floats from one staged chunk of a row of A to the next

// v = p[k .. k + 3], zeros where the row or k is outside; no branch: an address that is outside is replaced by the
// row's first element, which is always there.
template <typename TA, bool VEC>
__device__ __forceinline__ void fetch4(const TA* p, int k, int K, bool row_ok, float (&v)[4]) {
  if (VEC) {
    const bool ok = row_ok && k < K;         // K is a multiple of 4 here
    load4(p + (ok ? k : 0), v);
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = ok ? v[i] : 0.f;
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = row_ok && k + i < K;
      const float x = to_float(p[ok ? k + i : 0]);
      v[i] = ok ? x : 0.f;
    }
  }
}

template <typename TA, typename TC, int MT, int SCH, bool VEC>
__global__ __launch_bounds__(512) void gemm_nt_stream_kernel(const TA* __restrict__ A, int64_t lda,
                                                             const TA* __restrict__ W, int64_t ldw,
                                                             TC* __restrict__ C, int64_t ldc, int M, int N, int K,
                                                             int R) {
  extern __shared__ float lds[];
  float* As = lds;                            // [MT][SCH][SPAD]
  float* part = lds + MT * SCH * SPAD;        // [SCH][R][MT]: the chunks' sums of the running block
  const int tid = threadIdx.x;
  const int c = tid % SCH, r = tid / SCH;
  const int n = blockIdx.x * R + r;
  const bool n_ok = n < N;
  const TA* wrow = W + (int64_t)(n_ok ? n : 0) * ldw;
  // the result element that this thread finishes (threads 0 .. R * MT - 1)
  static_assert(MT <= SCH, "R * MT result elements over R * SCH threads");
  const int fr = tid / MT, fm = tid % MT;
  const bool finisher = tid < R * MT;
  float tot = 0.f;
  for (int kb = 0; kb < K; kb += SCH * CHUNK_K) {
    // The block of A into LDS, rows beyond M as zeros: 8 loads of 16 bytes of a thread on their way at a time.  This
    // thread's weights of the block are asked for behind the last of them and before anything waits: loads come back
    // in the order they were asked for, so A (small, shared by every workgroup, from the caches) is staged and the
    // first products run while the later weights are still on their way from memory.
    float wv[CHUNK_K / 4][4];
    constexpr int ITEMS = MT * SCH * (CHUNK_K / 4);       // at least 4 a thread: MT >= 4, R <= 16
    const int stride = 8 * blockDim.x;
    const int last = tid + (ITEMS - 1 - tid) / stride * stride;      // where this thread's last batch begins
    float v[8][4];
    auto ask = [&](int base) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = base + u * blockDim.x;
        const int idc = idx < ITEMS ? idx : 0;
        const int m = idc / (SCH * (CHUNK_K / 4)), q = idc % (SCH * (CHUNK_K / 4));
        fetch4<TA, VEC>(A + (int64_t)(m < M ? m : 0) * lda, kb + 4 * q, K, m < M, v[u]);
      }
    };
    auto stage = [&](int base) {
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int idx = base + u * blockDim.x;
        if (idx < ITEMS) {
          const int m = idx / (SCH * (CHUNK_K / 4)), q = idx % (SCH * (CHUNK_K / 4));
          store4(As + (m * SCH + q / (CHUNK_K / 4)) * SPAD + 4 * (q % (CHUNK_K / 4)), v[u]);
        }
      }
    };
    for (int base = tid; base < last; base += stride) {
      ask(base);
      stage(base);
    }
    ask(last);
#pragma unroll
    for (int q = 0; q < CHUNK_K / 4; ++q) fetch4<TA, VEC>(wrow, kb + c * CHUNK_K + 4 * q, K, n_ok, wv[q]);
    stage(last);
    __syncthreads();
    float acc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m] = 0.f;
#pragma unroll
    for (int q = 0; q < CHUNK_K / 4; ++q) {
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        float a[4];
        load4(As + (m * SCH + c) * SPAD + 4 * q, a);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[m] = fmaf(a[i], wv[q][i], acc[m]);
      }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m) part[(c * R + r) * MT + m] = acc[m];
    __syncthreads();
    if (finisher) {
      const int chunks = min(SCH, (K - kb + CHUNK_K - 1) / CHUNK_K);
      for (int cc = 0; cc < chunks; ++cc) tot += part[(cc * R + fr) * MT + fm];
    }
    // (the next block's first barrier keeps its writes to `part` behind these reads)
  }
  const int fn = blockIdx.x * R + fr;
  if (finisher && fm < M && fn < N) C[(int64_t)fm * ldc + fn] = from_float<TC>(tot);
}

// The same product for up to 8 rows of 32-bit A where all of k fits LDS beside R rows of W (k a multiple of 256) and
// the row groups make at most one workgroup for every compute unit: both operands go straight from memory to LDS
// (global_load_lds: lane i's 16 bytes land at base + 16 i), every load instruction of a wave covering 1 KB of one
// row, which the per-thread loads of the kernel above do not (a thread there walks its own 256 bytes, so an
// instruction touches 64 lines of memory: 2 TB/s).  A chunk's 16 pieces of 16 bytes are stored rotated by the
// chunk's number (piece q of chunk c at place (q + c) mod 16), so that the threads of different chunks, which read
// piece q at the same time, find theirs in different banks.  Thread (row pair, half of A's rows, chunk) then runs
// the chunk chains of 2 rows of W against 4 rows of A (6 reads of LDS for 32 multiply-adds, where a thread with one
// row of W and all rows of A needs 9), k ascending from zero as everywhere; the chunks' sums go through LDS to one
// thread per result element, which adds them in order.  Rows of A beyond M repeat row M - 1 and rows of W beyond N
// repeat row N - 1 (loads to LDS cannot be replaced by zeros); their results are not stored.
#define LDS_MT 8
__global__ __launch_bounds__(512) void gemm_nt_lds_kernel(const float* __restrict__ A, int64_t lda,
                                                          const float* __restrict__ W, int64_t ldw,
                                                          float* __restrict__ C, int64_t ldc, int M, int N, int K, int R) {
  extern __shared__ float lds[];
  const int SCH = K >> 6, UPR = SCH >> 2;      // chunks of a row; wave loads (1 KB: 4 chunks) of a row
  float* Ws = lds;                             // [R][K]
  float* As = lds + R * K;                     // [LDS_MT][K]
  float* part = As + LDS_MT * K;               // [SCH][R][LDS_MT]
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6), waves = blockDim.x >> 6;
  const int n0 = blockIdx.x * R;
  const int lc = lane >> 4, place = lane & 15;
  // A first: it comes from the caches and is there when the weights arrive
  for (int i = wave; i < LDS_MT * UPR; i += waves) {
    const int m = i / UPR, c = (i - m * UPR) * 4 + lc;
    const float* src = A + (int64_t)min(m, M - 1) * lda + c * 64 + ((place - c) & 15) * 4;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(As + i * 256), 16, 0, 0);
  }
  for (int i = wave; i < R * UPR; i += waves) {
    const int r = i / UPR, c = (i - r * UPR) * 4 + lc;
    const float* src = W + (int64_t)min(n0 + r, N - 1) * ldw + c * 64 + ((place - c) & 15) * 4;
    __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)src,
                                     (__attribute__((address_space(3))) void*)(Ws + i * 256), 16, 0, 0);
  }
  // the compiler does not count the requests that write LDS: the wait is written out
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  const int c = tid % SCH, mh = (tid / SCH) & 1, rp = tid / (2 * SCH);
  float acc[2][4];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int m = 0; m < 4; ++m) acc[a][m] = 0.f;
  const float* w0 = Ws + (2 * rp) * K + c * 64;
  const float* w1 = w0 + K;
  const float* a0 = As + (4 * mh) * K + c * 64;
#pragma unroll
  for (int q = 0; q < CHUNK_K / 4; ++q) {
    const int at = ((q + c) & 15) * 4;
    float wa[4], wb[4];
    load4(w0 + at, wa);
    load4(w1 + at, wb);
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      float a[4];
      load4(a0 + m * K + at, a);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc[0][m] = fmaf(a[i], wa[i], acc[0][m]);
        acc[1][m] = fmaf(a[i], wb[i], acc[1][m]);
      }
    }
  }
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int m = 0; m < 4; ++m) part[(c * R + 2 * rp + a) * LDS_MT + 4 * mh + m] = acc[a][m];
  __syncthreads();
  for (int f = tid; f < R * LDS_MT; f += blockDim.x) {
    const int fr = f / LDS_MT, fm = f - fr * LDS_MT;
    float tot = 0.f;
    for (int x = 0; x < SCH; ++x) tot += part[(x * R + fr) * LDS_MT + fm];
    if (fm < M && n0 + fr < N) C[(int64_t)fm * ldc + n0 + fr] = tot;
  }
}

static int gemm_compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
  }
  return cus;
}

template <typename TA, typename TC, int MT, int SCH, bool VEC>
static int launch_stream_instance(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M,
                                  int N, int K, int R, hipStream_t stream) {
  const size_t lds = ((size_t)MT * SCH * SPAD + (size_t)SCH * R * MT) * sizeof(float);
  static bool raised = false;       // per instantiation: more dynamic LDS than the default allotment
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_nt_stream_kernel<TA, TC, MT, SCH, VEC>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    MI_REQUIRE(e == hipSuccess, "gemm_nt: cannot raise the LDS allotment: %s", hipGetErrorString(e));
    raised = true;
  }
  gemm_nt_stream_kernel<TA, TC, MT, SCH, VEC><<<ceil_div(N, R), R * SCH, lds, stream>>>(
      (const TA*)A, lda, (const TA*)W, ldw, (TC*)C, ldc, M, N, K, R);
  return 0;
}

// Launches gemm_nt_lds_kernel where it is the quicker one (0), or says that the case is not its own (1): up to 8 rows
// of A, k a multiple of 256, 16-byte alignment, and a number of rows R of W per workgroup that fits LDS and with which
// the row groups do not exceed the compute units (a second round of such workgroups would wait for the first: nothing overlaps inside one).
// On an MI355X, 8 rows: [4096, 1024] 7.5 against 9.2 us, [1024, 2048] 7.2 against 9.7, [1024, 3072] 8.6 against 11.6;
// [6144, 1024] (384 row groups) 12.1 against 11.3, which is why it stays with the kernel above.
static int launch_lds(const float* A, int64_t lda, const float* W, int64_t ldw, float* C, int64_t ldc, int M, int N, int K,
                      int cus, hipStream_t stream) {
  if (M > LDS_MT || K % 256 != 0 || lda % 4 != 0 || ldw % 4 != 0 || (uintptr_t)A % 16 != 0 || (uintptr_t)W % 16 != 0) return 1;
  const int sch = K / CHUNK_K;
  // R: even, at least as many as leave no more row groups than compute units; 8 where fewer would do and 8 still
  // make a group for every other unit (fewer workgroups read A less often: [1024, 2048] 7.2 against 7.6 us with 4);
  // the first such R upwards whose workgroup is whole waves, up to 512 threads, and fits LDS, else the largest below
  int R = 0;
  size_t lds = 0;
  const int r_min = 2 * ceil_div(N, 2 * cus);
  const int r_want = (r_min < 8 && ceil_div(N, 8) >= cus / 2) ? 8 : r_min;
  auto fits = [&](int r, size_t* need) {
    *need = ((size_t)(r + LDS_MT) * K + (size_t)sch * r * LDS_MT) * sizeof(float);
    const int threads = r * sch;           // (r / 2 row pairs) x 2 halves of A's rows x chunks
    return *need <= 160 * 1024 && threads <= 512 && threads % 64 == 0;
  };
  for (int r = r_want; r <= 32 && R == 0; r += 2)
    if ((r == r_min || ceil_div(N, r) >= cus / 2) && fits(r, &lds)) R = r;
  for (int r = r_want - 2; r >= r_min && r >= 2 && R == 0; r -= 2)
    if (fits(r, &lds)) R = r;
  if (R == 0 || ceil_div(N, R) > cus) return 1;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_nt_lds_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) {
      snprintf(g_mi_error, sizeof(g_mi_error), "gemm_nt: cannot raise the LDS allotment: %s", hipGetErrorString(e));
      return -1;
    }
    raised = true;
  }
  gemm_nt_lds_kernel<<<ceil_div(N, R), R * sch, lds, stream>>>(A, lda, W, ldw, C, ldc, M, N, K, R);
  return 0;
}

template <typename TA, typename TC>
static int launch_stream(const void* A, int64_t lda, const void* W, int64_t ldw, void* C, int64_t ldc, int M, int N, int K,
                         hipStream_t stream) {
  // Chunks a workgroup works on side by side: all of k at once where the staged rows of A fit LDS (every load of the
  // product is then on its way together, which is what its time comes to when W is small), in steps of 16 chunks.
  // Rows of W per workgroup: 16 where that still makes a workgroup for every compute unit, else 8 where that makes
  // one for every other unit, else 4 (every workgroup stages the rows of A once, so more rows mean fewer reads of
  // A; what fills the machine is the bytes on their way, 256 of them a thread), and never more than 512 threads.
  const int cus = gemm_compute_units();
  if (std::is_same<TA, float>::value && std::is_same<TC, float>::value) {
    const int rc = launch_lds((const float*)A, lda, (const float*)W, ldw, (float*)C, ldc, M, N, K, cus, stream);
    if (rc <= 0) return -rc;      // 0: launched; negative: an error; 1: not its case
  }
  const int mt = M <= 4 ? 4 : (M <= 8 ? 8 : 16);
  const int chunks = ceil_div(K, CHUNK_K);
  int sch = chunks <= 16 ? 16 : (chunks <= 32 || mt == 16 ? 32 : 48);
  int R = N / 16 >= cus ? 16 : (N / 8 >= cus / 2 ? 8 : 4);
  while (R > 1 && (R * sch > 512 || ((size_t)mt * sch * SPAD + (size_t)sch * R * mt) * sizeof(float) > 160 * 1024)) R /= 2;
  const bool vec = K % 4 == 0 && lda % 4 == 0 && ldw % 4 == 0 && (uintptr_t)A % 16 == 0 && (uintptr_t)W % 16 == 0;
#define GO(MT, SCH)                                                                                                  \
  return vec ? launch_stream_instance<TA, TC, MT, SCH, true>(A, lda, W, ldw, C, ldc, M, N, K, R, stream)            \
             : launch_stream_instance<TA, TC, MT, SCH, false>(A, lda, W, ldw, C, ldc, M, N, K, R, stream)
  if (mt == 4) {
    if (sch == 16) GO(4, 16);
    if (sch == 32) GO(4, 32);
    GO(4, 48);
  }
  if (mt == 8) {
    if (sch == 16) GO(8, 16);
    if (sch == 32) GO(8, 32);
    GO(8, 48);
  }
  if (sch == 16) GO(16, 16);
  GO(16, 32);
#undef GO
}

// in_dtype: dtype of A and W; out_dtype: dtype of C.
MI_EXPORT int mi_gemm_nt(int in_dtype, int out_dtype, const void* A, int64_t lda, const void* W, int64_t ldw, void* C,
                         int64_t ldc, int M, int N, int K, hipStream_t stream) {
  MI_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_nt: bad sizes M=%d N=%d K=%d", M, N, K);
  MI_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_nt: leading dimensions (%lld, %lld, %lld) too small for K=%d N=%d",
             (long long)lda, (long long)ldw, (long long)ldc, K, N);
  if (M == 0) return 0;
  const bool few = M <= 16;
  dim3 grid(ceil_div(N, BN), ceil_div(M, BM));
  MI_REQUIRE(grid.y <= 65535, "gemm_nt: M=%d too large for one launch", M);
#define LAUNCH(TA, TC)                                                                                              \
  if (few) {                                                                                                        \
    const int rc = launch_stream<TA, TC>(A, lda, W, ldw, C, ldc, M, N, K, stream);                                  \
    if (rc) return rc;                                                                                              \
  } else                                                                                                            \
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
