// Next-token choice from 32-bit logits, one workgroup per row.
//
//   temperature == 0 : argmax, the lowest index wins a tie (torch.argmax, miniinfer/layers/sample.py:111-112)
//   temperature  > 0 : a draw from softmax(logits / temperature) (sample.py:115-128), optionally limited
//                      to the top_k most probable tokens and then to the smallest set of most probable
//                      tokens whose (renormalised) mass reaches top_p (sample.py:117-121; 0 / 1.0 disable).
//
// The draw is the Gumbel-max form of the reference's exponential race (sample.py:125-128):
// argmax_i( logit_i / T + G_i ), G_i = -log(-log(u_i)), with u_i from a counter-based generator keyed
// by (seed, step, i) per row, so a request's tokens do not depend on what else is in the batch.
// Tokens tied in value with the k-th largest, or with the top_p threshold, are all kept.
#include "common.h"

#define SAMPLE_THREADS 1024

__host__ __device__ __forceinline__ uint64_t mix64(uint64_t seed, uint64_t step, uint64_t i) {
  uint64_t z = (seed ^ (step * 0xD1B54A32D192ED03ull)) + (i + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float uniform01(uint64_t seed, uint64_t step, uint64_t i) {
  return ((float)(mix64(seed, step, i) >> 41) + 0.5f) * (1.0f / 8388608.0f);   // in (0, 1), exact in 32-bit
}

// order-preserving map of a float to an unsigned key (larger float = larger key)
__device__ __forceinline__ uint32_t ordered_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

struct ArgMax {
  float v;
  int i;
};

__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ __forceinline__ ArgMax block_argmax(ArgMax a, ArgMax* scratch) {
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int wave = threadIdx.x / MI_WAVE;
#pragma unroll
  for (int o = MI_WAVE / 2; o > 0; o >>= 1) {
    ArgMax b;
    b.v = __shfl_xor(a.v, o, MI_WAVE);
    b.i = __shfl_xor(a.i, o, MI_WAVE);
    a = better(a, b);
  }
  __syncthreads();
  if (lane == 0) scratch[wave] = a;
  __syncthreads();
  ArgMax r = scratch[0];
  for (int w = 1; w < SAMPLE_THREADS / MI_WAVE; ++w) r = better(r, scratch[w]);
  return r;
}

__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (MI_WAVE - 1);
  const int wave = threadIdx.x / MI_WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < SAMPLE_THREADS / MI_WAVE; ++w) r = fmaxf(r, scratch[w]);
  return r;
}

// Radix descent over the ordered keys of one row.  At each of 4 levels (8 bits, most significant first) a
// 256-bin histogram of `weight` is built over the elements that match the prefix found so far; bins are
// walked from the largest digit down until the running total reaches `target`.  On return, `prefix` is the
// key of the threshold element: total weight of keys > prefix is < target <= total weight of keys >= prefix.
// COUNT: weight 1 per element (k-th largest).  Otherwise weight exp(x - m) (probability mass), restricted
// to keys >= min_key.
template <bool COUNT>
__device__ uint32_t radix_threshold(const float* __restrict__ row, int V, float inv_t, float m, float target,
                                    uint32_t min_key, float* hist, uint32_t* shared_prefix, float* shared_above) {
  uint32_t prefix = 0;
  float above = 0.f;   // weight of keys strictly above the current prefix range
  for (int level = 0; level < 4; ++level) {
    const int shift = 24 - 8 * level;
    const uint32_t mask = level == 0 ? 0u : (0xffffffffu << (shift + 8));
    for (int b = threadIdx.x; b < 256; b += blockDim.x) hist[b] = 0.f;
    __syncthreads();
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i] * inv_t;
      const uint32_t key = ordered_key(x);
      if ((key & mask) == prefix && key >= min_key) {
        const float wgt = COUNT ? 1.f : expf(x - m);
        atomicAdd(&hist[(key >> shift) & 0xff], wgt);
      }
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      float run = above;
      int digit = 0;
      for (int b = 255; b >= 0; --b) {
        if (run + hist[b] >= target || b == 0) {
          digit = b;
          break;
        }
        run += hist[b];
      }
      *shared_prefix = prefix | ((uint32_t)digit << shift);
      *shared_above = run;
    }
    __syncthreads();
    prefix = *shared_prefix;
    above = *shared_above;
    __syncthreads();
  }
  return prefix;
}

__global__ __launch_bounds__(SAMPLE_THREADS) void sample_kernel(
    const float* __restrict__ logits, int64_t row_stride, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const uint64_t* __restrict__ seeds,
    const int64_t* __restrict__ steps, int* __restrict__ out) {
  __shared__ ArgMax am_scratch[SAMPLE_THREADS / MI_WAVE];
  __shared__ float f_scratch[SAMPLE_THREADS / MI_WAVE];
  __shared__ float hist[256];
  __shared__ uint32_t sh_prefix;
  __shared__ float sh_above;
  const int r = blockIdx.x;
  const float* row = logits + (int64_t)r * row_stride;
  const float temp = temperature ? temperature[r] : 0.f;

  if (!(temp > 0.f)) {
    ArgMax a = {-INFINITY, V};
    for (int i = threadIdx.x; i < V; i += blockDim.x) a = better(a, ArgMax{row[i], i});
    a = block_argmax(a, am_scratch);
    if (threadIdx.x == 0) out[r] = a.i < V ? a.i : 0;
    return;
  }

  const float inv_t = 1.f / temp;
  const int k = top_k ? top_k[r] : 0;
  const float p = top_p ? top_p[r] : 1.f;
  uint32_t min_key = 0;   // tokens whose key is below this are filtered out
  if (k > 0 && k < V) {
    min_key = radix_threshold<true>(row, V, inv_t, 0.f, (float)k, 0u, hist, &sh_prefix, &sh_above);
  }
  if (p < 1.f) {
    float m = -INFINITY;
    for (int i = threadIdx.x; i < V; i += blockDim.x) m = fmaxf(m, row[i] * inv_t);
    m = block_max(m, f_scratch);
    float z = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float x = row[i] * inv_t;
      if (ordered_key(x) >= min_key) z += expf(x - m);
    }
    z = block_sum(z, f_scratch);
    const uint32_t key = radix_threshold<false>(row, V, inv_t, m, p * z, min_key, hist, &sh_prefix, &sh_above);
    if (key > min_key) min_key = key;
  }
  const uint64_t seed = seeds ? seeds[r] : 0;
  const uint64_t step = steps ? (uint64_t)steps[r] : 0;
  ArgMax a = {-INFINITY, V};
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    const float x = row[i] * inv_t;
    if (ordered_key(x) < min_key) continue;
    const float u = uniform01(seed, step, (uint64_t)i);
    const float g = -logf(-logf(u));
    a = better(a, ArgMax{x + g, i});
  }
  a = block_argmax(a, am_scratch);
  if (threadIdx.x == 0) out[r] = a.i < V ? a.i : 0;
}

// ---------------------------------------------------------------- rows without top_k / top_p: the vocabulary in parts
// Stage 1: block (part, row) finds the best (value, index) of its part of the vocabulary, value = logit for a greedy
// row and logit / T + Gumbel noise for a sampled one.  Stage 2: one wave per row picks the best part.
#define PART_THREADS 256
#define PART_ELEMS 4096

__global__ __launch_bounds__(PART_THREADS) void sample_parts_kernel(
    const float* __restrict__ logits, int64_t row_stride, int V, const float* __restrict__ temperature,
    const uint64_t* __restrict__ seeds, const int64_t* __restrict__ steps, float* __restrict__ part_val,
    int* __restrict__ part_idx) {
  __shared__ ArgMax scratch[PART_THREADS / MI_WAVE];
  const int r = blockIdx.y, part = blockIdx.x, nparts = gridDim.x;
  const float* row = logits + (int64_t)r * row_stride;
  const float temp = temperature ? temperature[r] : 0.f;
  const bool greedy = !(temp > 0.f);
  const float inv_t = greedy ? 1.f : 1.f / temp;
  const uint64_t seed = seeds ? seeds[r] : 0;
  const uint64_t step = steps ? (uint64_t)steps[r] : 0;
  const int begin = part * PART_ELEMS;
  const int end = min(V, begin + PART_ELEMS);
  ArgMax a = {-INFINITY, V};
  for (int i = begin + threadIdx.x; i < end; i += PART_THREADS) {
    float x = row[i];
    if (!greedy) x = x * inv_t - logf(-logf(uniform01(seed, step, (uint64_t)i)));
    a = better(a, ArgMax{x, i});
  }
  const int lane = threadIdx.x & (MI_WAVE - 1), wave = threadIdx.x / MI_WAVE;
#pragma unroll
  for (int o = MI_WAVE / 2; o > 0; o >>= 1) {
    ArgMax b;
    b.v = __shfl_xor(a.v, o, MI_WAVE);
    b.i = __shfl_xor(a.i, o, MI_WAVE);
    a = better(a, b);
  }
  if (lane == 0) scratch[wave] = a;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < PART_THREADS / MI_WAVE; ++w) a = better(a, scratch[w]);
    part_val[(int64_t)r * nparts + part] = a.v;
    part_idx[(int64_t)r * nparts + part] = a.i;
  }
}

__global__ __launch_bounds__(MI_WAVE) void sample_pick_kernel(const float* __restrict__ part_val,
                                                              const int* __restrict__ part_idx, int nparts, int V,
                                                              int* __restrict__ out) {
  const int r = blockIdx.x;
  ArgMax a = {-INFINITY, V};
  for (int p = threadIdx.x; p < nparts; p += MI_WAVE)
    a = better(a, ArgMax{part_val[(int64_t)r * nparts + p], part_idx[(int64_t)r * nparts + p]});
#pragma unroll
  for (int o = MI_WAVE / 2; o > 0; o >>= 1) {
    ArgMax b;
    b.v = __shfl_xor(a.v, o, MI_WAVE);
    b.i = __shfl_xor(a.i, o, MI_WAVE);
    a = better(a, b);
  }
  if (threadIdx.x == 0) out[r] = a.i < V ? a.i : 0;
}

MI_EXPORT int mi_sample_parts_count(int V) { return (V + PART_ELEMS - 1) / PART_ELEMS; }

// Greedy and plain temperature rows (no top_k, no top_p).  part_val / part_idx: scratch of R * mi_sample_parts_count(V).
MI_EXPORT int mi_sample_simple(const float* logits, int64_t row_stride, int R, int V, const float* temperature,
                               const uint64_t* seeds, const int64_t* steps, float* part_val, int* part_idx, int* out,
                               hipStream_t stream) {
  MI_REQUIRE(R >= 0 && V > 0 && row_stride >= V, "sample: bad sizes R=%d V=%d stride=%lld", R, V, (long long)row_stride);
  MI_REQUIRE(R <= 65535, "sample: %d rows are too many for one launch", R);
  MI_REQUIRE(part_val && part_idx, "sample: no scratch");
  if (R == 0) return 0;
  const int nparts = (V + PART_ELEMS - 1) / PART_ELEMS;
  sample_parts_kernel<<<dim3(nparts, R), PART_THREADS, 0, stream>>>(logits, row_stride, V, temperature, seeds, steps,
                                                                    part_val, part_idx);
  MI_CHECK_LAUNCH("sample parts");
  sample_pick_kernel<<<R, MI_WAVE, 0, stream>>>(part_val, part_idx, nparts, V, out);
  MI_CHECK_LAUNCH("sample pick");
  return 0;
}

MI_EXPORT int mi_sample(const float* logits, int64_t row_stride, int R, int V, const float* temperature,
                        const int* top_k, const float* top_p, const uint64_t* seeds, const int64_t* steps, int* out,
                        hipStream_t stream) {
  MI_REQUIRE(R >= 0 && V > 0 && row_stride >= V, "sample: bad sizes R=%d V=%d stride=%lld", R, V, (long long)row_stride);
  if (R == 0) return 0;
  sample_kernel<<<R, SAMPLE_THREADS, 0, stream>>>(logits, row_stride, V, temperature, top_k, top_p, seeds, steps, out);
  MI_CHECK_LAUNCH("sample");
  return 0;
}

// host twin of the generator, for tests: u[i] for i in [0, n)
MI_EXPORT void mi_sample_uniforms_host(uint64_t seed, uint64_t step, int n, float* u) {
  for (int i = 0; i < n; ++i) u[i] = ((float)(mix64(seed, step, (uint64_t)i) >> 41) + 0.5f) * (1.0f / 8388608.0f);
}
