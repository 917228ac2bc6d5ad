// Token choice from float logits [M, V], one block per row.
//   temperature[r] <= 0 : greedy, the lowest index among the maxima;
//   temperature[r] >  0 : a draw from softmax(logits / temperature) by the Gumbel-max
//     rule: argmax_i( logits[i] / T + g_i ), g_i = -log(-log(u_i)), where u_i in (0,1)
//     comes from a counter-based generator keyed by (key[r], i).  The draw depends on
//     the row's key and logits only, not on the batch it is in.
#include "common.h"

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float uniform_open01(uint64_t key, uint32_t i) {
  const uint64_t bits = mix64(mix64(key) ^ (uint64_t)i * 0xD1342543DE82EF95ull);
  // 24 high bits -> (0, 1): never 0, never 1
  return ((float)(bits >> 40) + 0.5f) * (1.0f / 16777216.0f);
}

__global__ void __launch_bounds__(256)
sample_kernel(int* __restrict__ out, const float* __restrict__ logits, long long row_stride, int V,
              const float* __restrict__ temperature, const unsigned long long* __restrict__ keys) {
  __shared__ float bv[4];
  __shared__ int bi[4];
  const long long r = blockIdx.x;
  const float* row = logits + r * row_stride;
  const float temp = temperature ? temperature[r] : 0.f;
  const uint64_t key = keys ? keys[r] : 0ull;
  const float inv_t = temp > 0.f ? 1.f / temp : 1.f;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    float v = row[i] * inv_t;
    if (temp > 0.f) {
      const float u = uniform_open01(key, (uint32_t)i);
      v += -logf(-logf(u));
    }
    if (v > best || (v == best && i < best_i)) { best = v; best_i = i; }
  }
  // NaN logits never win a comparison; a row of them yields index 0x7fffffff -> reported as V
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (ov > best || (ov == best && oi < best_i)) { best = ov; best_i = oi; }
  }
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  if (lane == 0) { bv[wid] = best; bi[wid] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < best_i)) { best = bv[w]; best_i = bi[w]; }
    out[r] = best_i < V ? best_i : V;
  }
}

extern "C" int jv_sample(int* out, const float* logits, long long row_stride, int n_rows, int V,
                         const float* temperature, const unsigned long long* keys, void* stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(256), 0, (hipStream_t)stream, out, logits,
                     row_stride, V, temperature, keys);
  return JV_LAUNCH_CHECK();
}
