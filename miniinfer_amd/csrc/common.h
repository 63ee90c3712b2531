// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of this library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#define MI_WAVE 64

// ---------------------------------------------------------------- error reporting (host)
// Every entry point returns 0 on success; otherwise the message is read with mi_last_error().
static thread_local char g_mi_error[512] = {0};

#define MI_FAIL(...)                                            \
  do {                                                          \
    snprintf(g_mi_error, sizeof(g_mi_error), __VA_ARGS__);      \
    return 1;                                                   \
  } while (0)

#define MI_REQUIRE(cond, ...) \
  do {                        \
    if (!(cond)) MI_FAIL(__VA_ARGS__); \
  } while (0)

#define MI_CHECK_LAUNCH(name)                                                   \
  do {                                                                          \
    hipError_t e_ = hipGetLastError();                                          \
    if (e_ != hipSuccess) MI_FAIL("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

#define MI_EXPORT extern "C" __attribute__((visibility("default")))

// ---------------------------------------------------------------- bfloat16 as raw bits
struct bf16 {
  uint16_t bits;
};

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}

// round to nearest even; NaN stays NaN
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16 x) { return bf16_bits_to_float(x.bits); }

// two values of the activation dtype at once (a 32-bit or 64-bit access)
typedef __bf16 mi_bf16x2 __attribute__((ext_vector_type(2)));
typedef float mi_f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void load2(const float* p, float& a, float& b) {
  const mi_f32x2 v = *reinterpret_cast<const mi_f32x2*>(p);
  a = v[0];
  b = v[1];
}
__device__ __forceinline__ void load2(const bf16* p, float& a, float& b) {
  const uint32_t u = *reinterpret_cast<const uint32_t*>(p);
  a = __uint_as_float(u << 16);
  b = __uint_as_float(u & 0xffff0000u);
}
__device__ __forceinline__ void store2(float* p, float a, float b) {
  *reinterpret_cast<mi_f32x2*>(p) = mi_f32x2{a, b};
}
__device__ __forceinline__ void store2(bf16* p, float a, float b) {   // v_cvt_pk_bf16_f32: round to nearest even
  const mi_f32x2 v = {a, b};
  const mi_bf16x2 r = __builtin_convertvector(v, mi_bf16x2);
  *reinterpret_cast<uint32_t*>(p) = *reinterpret_cast<const uint32_t*>(&r);
}

// four values at once (a 64-bit or 128-bit access)
typedef float mi_f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t mi_u32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ void load4(const float* p, float (&v)[4]) {
  const mi_f32x4 x = *reinterpret_cast<const mi_f32x4*>(p);
  v[0] = x[0];
  v[1] = x[1];
  v[2] = x[2];
  v[3] = x[3];
}
__device__ __forceinline__ void load4(const bf16* p, float (&v)[4]) {
  const mi_u32x2 u = *reinterpret_cast<const mi_u32x2*>(p);
  v[0] = __uint_as_float(u[0] << 16);
  v[1] = __uint_as_float(u[0] & 0xffff0000u);
  v[2] = __uint_as_float(u[1] << 16);
  v[3] = __uint_as_float(u[1] & 0xffff0000u);
}
__device__ __forceinline__ void store4(float* p, const float (&v)[4]) {
  *reinterpret_cast<mi_f32x4*>(p) = mi_f32x4{v[0], v[1], v[2], v[3]};
}
__device__ __forceinline__ void store4(bf16* p, const float (&v)[4]) {
  const mi_f32x2 lo = {v[0], v[1]}, hi = {v[2], v[3]};
  const mi_bf16x2 a = __builtin_convertvector(lo, mi_bf16x2), b = __builtin_convertvector(hi, mi_bf16x2);
  *reinterpret_cast<mi_u32x2*>(p) = mi_u32x2{*reinterpret_cast<const uint32_t*>(&a), *reinterpret_cast<const uint32_t*>(&b)};
}

template <typename T>
__device__ __forceinline__ T from_float(float x);
template <>
__device__ __forceinline__ float from_float<float>(float x) { return x; }
template <>
__device__ __forceinline__ bf16 from_float<bf16>(float x) {
  bf16 r;
  r.bits = float_to_bf16_bits(x);
  return r;
}

// ---------------------------------------------------------------- reductions
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = MI_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, MI_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = MI_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MI_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; `scratch` holds 16 floats of LDS. Every thread gets the sum.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int wave = threadIdx.x / MI_WAVE;
  const int nwaves = (blockDim.x + MI_WAVE - 1) / MI_WAVE;
  v = wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nwaves; ++i) t += scratch[i];
  return t;
}

static inline int ceil_div(int64_t a, int64_t b) { return (int)((a + b - 1) / b); }

// one translation unit per shared object: each exports its own message reader
MI_EXPORT const char* mi_last_error() { return g_mi_error; }

#define MI_DTYPE_F32 0
#define MI_DTYPE_BF16 1
