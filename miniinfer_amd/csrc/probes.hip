// Two measuring kernels that do nothing useful: what this GPU delivers when a kernel only reads memory, and when
// it only feeds the matrix cores.  The benchmark prices the engine's steps against these measured figures beside
// the data sheet's (8 TB/s, 2.5 PFLOP/s dense bfloat16).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Every workgroup reads a contiguous slice of the buffer, 16 bytes a lane and UNROLL loads in flight, and xors what
// it read into one word, which is stored only if it has a value that random data practically never gives (the
// compiler must keep the loads, memory sees no write traffic).  (Slices per workgroup stream faster than one
// stride of the whole grid: 6.2 against 5.8 TB/s.)
template <int UNROLL>
__global__ __launch_bounds__(256) void stream_read_kernel(const u32x4* __restrict__ src, int64_t n16,
                                                          uint32_t* __restrict__ sink) {
  const int64_t per_block = (n16 + gridDim.x - 1) / gridDim.x;
  const int64_t begin = (int64_t)blockIdx.x * per_block;
  const int64_t end = begin + per_block < n16 ? begin + per_block : n16;
  int64_t i = begin + threadIdx.x;
  u32x4 acc = {0, 0, 0, 0};
  for (; i + (UNROLL - 1) * 256 < end; i += UNROLL * 256) {
    u32x4 v[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) v[u] = src[i + u * 256];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) acc ^= v[u];
  }
  for (; i < end; i += 256) acc ^= src[i];
  const uint32_t x = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
  if (x == 0x9e3779b9u) sink[0] = x;
}

// src: `bytes` bytes (a multiple of 16) of device memory; sink: one word.
MI_EXPORT int mi_probe_stream_read(const void* src, int64_t bytes, void* sink, hipStream_t stream) {
  MI_REQUIRE(src && sink && bytes >= 16 && bytes % 16 == 0, "probe_stream_read: bytes=%lld", (long long)bytes);
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  stream_read_kernel<16><<<cus * 8, 256, 0, stream>>>((const u32x4*)src, bytes / 16, (uint32_t*)sink);
  MI_CHECK_LAUNCH("probe_stream_read");
  return 0;
}

// Each wave runs `iters` rounds of CHAINS independent 32x32x16 bfloat16 products on operands that never leave its
// registers; the accumulators are stored at the end only if they hold a value they cannot hold.
constexpr int CHAINS = 4;
__global__ __launch_bounds__(256) void mfma_loop_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 7));
    b[i] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
  }
  f32x16 acc[CHAINS];
#pragma unroll
  for (int c = 0; c < CHAINS; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[c][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int c = 0; c < CHAINS; ++c) acc[c] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[c], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < CHAINS; ++c)
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[c][i];
  if (s == -1.f) sink[0] = s;
}

// Launches blocks * 4 waves of `iters` rounds; *flops receives the floating-point operations of the launch.
MI_EXPORT int mi_probe_mfma(int blocks, int iters, void* sink, double* flops, hipStream_t stream) {
  MI_REQUIRE(blocks > 0 && iters > 0 && sink, "probe_mfma: blocks=%d iters=%d", blocks, iters);
  mfma_loop_kernel<<<blocks, 256, 0, stream>>>(iters, (float*)sink);
  MI_CHECK_LAUNCH("probe_mfma");
  if (flops) *flops = (double)blocks * 4.0 * (double)iters * CHAINS * (2.0 * 32 * 32 * 16);
  return 0;
}
