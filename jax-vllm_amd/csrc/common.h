// Shared device helpers for the gfx950 (CDNA4, wave64) kernels of this library.
//
// Conventions of every exported entry point (extern "C", prefix jv_):
//   * raw device pointers, sizes as int / long long, the HIP stream last as void*;
//   * returns the hipError_t of the launch as int (0 = success), launches nothing
//     when a size is zero, and allocates nothing;
//   * element types: "bf16" entry points take __bf16 activations and weights,
//     "f32" entry points take float; reductions, softmax, norms and rotation
//     angles are float in both.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define JV_WAVE 64

typedef __bf16 bf16_t;

template <typename T> __device__ __forceinline__ float to_f32(T x) { return (float)x; }
template <typename T> __device__ __forceinline__ T from_f32(float x) { return (T)x; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = JV_WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, JV_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = JV_WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, JV_WAVE));
  return v;
}

// Sum over a whole block of up to 1024 threads; `red` is shared scratch of >= 17 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE;
  const int nw = (blockDim.x + JV_WAVE - 1) / JV_WAVE;
  v = wave_sum(v);
  __syncthreads();  // protects `red` against a previous use
  if (lane == 0) red[wid] = v;
  __syncthreads();
  float t = (lane < nw) ? red[lane] : 0.f;
  t = wave_sum(t);
  return t;
}

#define JV_LAUNCH_CHECK() ((int)hipGetLastError())
