// What this chip delivers when nothing else is in the way: a kernel that only reads memory and a
// kernel that only feeds the matrix cores.  The measurement program times them beside the engine,
// so that its fractions of the published peaks (8 TB/s, 2.5 PFLOP/s dense bf16) can be read against
// what a plain streaming read and a plain MFMA loop reach on the same box.
#include "common.h"

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));

// Every block reads one contiguous share of the buffer, 16 bytes a lane, 8 loads in flight a lane.
// The sum is stored only if it has a value that zeros and finite data never give, so the loads stay.
__global__ void __launch_bounds__(256) calibrate_read_kernel(const f32x4* __restrict__ p, long long per_block,
                                                              float* __restrict__ sink) {
  const f32x4* q = p + (long long)blockIdx.x * per_block;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  long long i = threadIdx.x;
  for (; i + 7 * 256 < per_block; i += 8 * 256) {
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = q[i + u * 256];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  for (; i < per_block; i += 256) acc += q[i];
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) sink[0] = 1.f;
}

// Every wave keeps four independent 32x32 accumulators and issues v_mfma_f32_32x32x16_bf16 on
// operands that never leave its registers: 4 * 2 * 32 * 32 * 16 flops a turn of the loop.
__global__ void __launch_bounds__(256) calibrate_mfma_kernel(float* __restrict__ sink, int turns) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (__bf16)(0.001f * (float)((threadIdx.x + i) & 7));
    b[i] = (__bf16)(0.002f * (float)((threadIdx.x * 3 + i) & 7));
  }
  f32x16 c0 = {}, c1 = {}, c2 = {}, c3 = {};
  for (int t = 0; t < turns; ++t) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, a, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, a, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b, b, c3, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 16; ++i) s += c0[i] + c1[i] + c2[i] + c3[i];
  if (s == 12345.678f) sink[0] = s;
}

// Reads `bytes` (a multiple of 16) from p with `blocks` blocks of 256 threads.
extern "C" int jv_calibrate_read(const void* p, long long bytes, float* sink, int blocks, void* stream) {
  if (bytes <= 0 || blocks <= 0 || bytes % 16 != 0 || (bytes / 16) % blocks != 0) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(calibrate_read_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, (const f32x4*)p,
                     bytes / 16 / blocks, sink);
  return JV_LAUNCH_CHECK();
}

// `blocks` blocks of 4 waves, `turns` turns each; the flops done are jv_calibrate_mfma_flops(blocks, turns).
extern "C" int jv_calibrate_mfma(float* sink, int turns, int blocks, void* stream) {
  if (turns <= 0 || blocks <= 0) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(calibrate_mfma_kernel, dim3(blocks), dim3(256), 0, (hipStream_t)stream, sink, turns);
  return JV_LAUNCH_CHECK();
}

extern "C" double jv_calibrate_mfma_flops(int blocks, int turns) {
  return (double)blocks * 4.0 * (double)turns * 4.0 * 2.0 * 32.0 * 32.0 * 16.0;
}
