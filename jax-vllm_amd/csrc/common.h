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

// Gate activations of a gated feed-forward, y = act(gate) * up, in float.  The ids are part of the
// exported interface (the Python side names them).
#define JV_ACT_SILU 1        // gate / (1 + exp(-gate))
#define JV_ACT_GELU_TANH 2   // 0.5 gate (1 + tanh(sqrt(2/pi) (gate + 0.044715 gate^3)))
__host__ __device__ __forceinline__ bool jv_act_known(int act) { return act == JV_ACT_SILU || act == JV_ACT_GELU_TANH; }
__device__ __forceinline__ float jv_gated(int act, float gate, float up) {
  if (act == JV_ACT_GELU_TANH) {
    const float inner = 0.7978845608028654f * (gate + 0.044715f * gate * gate * gate);
    return 0.5f * gate * (1.f + tanhf(inner)) * up;
  }
  return gate / (1.f + expf(-gate)) * up;
}

#define JV_LAUNCH_CHECK() ((int)hipGetLastError())
