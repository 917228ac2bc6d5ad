// Embedding gather, fused residual-add + RMSNorm, plain RMSNorm, SiLU-mul.
// The residual stream is float in every mode; normalised outputs are in the
// activation type T.  All reductions are float.
#include "common.h"

// ---------------------------------------------------------------- embedding gather
// h[t, :] = float(table[ids[t], :]).  One block per token.
template <typename T>
__global__ void embedding_kernel(float* __restrict__ h, const T* __restrict__ table,
                                 const int* __restrict__ ids, int hidden) {
  const long long t = blockIdx.x;
  const T* row = table + (long long)ids[t] * hidden;
  float* out = h + t * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) out[i] = to_f32(row[i]);
}

// ---------------------------------------------------------------- residual add + RMSNorm
// Row r = rows ? rows[i] : i.
//   x = h[r] + (delta ? delta[r] : 0)            (float)
//   if (!rows) h[r] = x                          (residual stream updated in place)
//   out[i] = T( x * rsqrt(mean(x^2) + eps) * w )
// With `rows` given the residual stream is left untouched (used to norm only the
// rows whose logits are wanted).  One block per output row.
template <typename T>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                   const float* __restrict__ w, T* __restrict__ out,
                                   const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float red[32];
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  float* hr = h + r * hidden;
  const T* dr = delta ? delta + r * hidden : nullptr;
  T* o = out + i * hidden;
  float ss = 0.f;
  // pass 1: sum of squares (and the in-place residual update)
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float x = hr[c];
    if (dr) x += to_f32(dr[c]);
    if (!rows && dr) hr[c] = x;
    ss += x * x;
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)hidden + eps);
  // pass 2: the row is re-read (it is cache-resident); with `rows` the sum is redone
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    float x = hr[c];
    if (rows && dr) x += to_f32(dr[c]);
    o[c] = from_f32<T>(x * inv * w[c]);
  }
}

// ---------------------------------------------------------------- plain RMSNorm over the last axis
// out[r, :] = T( x[r,:] * rsqrt(mean(x^2)+eps) * w ), x of type T, rows of length n.
// One wave per row, several rows per block.
template <typename T>
__global__ void rmsnorm_kernel(T* __restrict__ out, const T* __restrict__ x,
                               const float* __restrict__ w, long long rows, int n, float eps) {
  const int lane = threadIdx.x & (JV_WAVE - 1);
  const long long r = (long long)blockIdx.x * (blockDim.x / JV_WAVE) + threadIdx.x / JV_WAVE;
  if (r >= rows) return;
  const T* xr = x + r * n;
  T* o = out + r * n;
  float ss = 0.f;
  for (int c = lane; c < n; c += JV_WAVE) {
    float v = to_f32(xr[c]);
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float inv = rsqrtf(ss / (float)n + eps);
  for (int c = lane; c < n; c += JV_WAVE) o[c] = from_f32<T>(to_f32(xr[c]) * inv * w[c]);
}

// ---------------------------------------------------------------- SiLU-mul
// out[t, j] = silu(gu[t, j]) * gu[t, inter + j], silu(x) = x / (1 + exp(-x)), in float.
template <typename T>
__global__ void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, long long total,
                                int inter) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  for (long long e = (long long)blockIdx.x * blockDim.x + threadIdx.x; e < total; e += stride) {
    const long long t = e / inter;
    const int j = (int)(e - t * inter);
    const float g = to_f32(gu[t * 2 * inter + j]);
    const float u = to_f32(gu[t * 2 * inter + inter + j]);
    out[e] = from_f32<T>(g / (1.f + expf(-g)) * u);
  }
}

// ---------------------------------------------------------------- float -> T copy of selected rows
template <typename T>
__global__ void cast_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                 const int* __restrict__ rows, int n) {
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  for (int c = threadIdx.x; c < n; c += blockDim.x) out[i * n + c] = from_f32<T>(x[r * n + c]);
}

#define DEFINE_ELEMENTWISE(SUF, T)                                                                  \
  extern "C" int jv_embedding_##SUF(float* h, const void* table, const int* ids, int n_tokens,      \
                                    int hidden, void* stream) {                                     \
    if (n_tokens <= 0) return 0;                                                                    \
    hipLaunchKernelGGL(embedding_kernel<T>, dim3(n_tokens), dim3(256), 0, (hipStream_t)stream, h,   \
                       (const T*)table, ids, hidden);                                               \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_add_rmsnorm_##SUF(float* h, const void* delta, const float* w, void* out,       \
                                      const int* rows, int n_out, int hidden, float eps,            \
                                      void* stream) {                                               \
    if (n_out <= 0) return 0;                                                                       \
    const int threads = hidden >= 2048 ? 512 : 256;                                                 \
    hipLaunchKernelGGL(add_rmsnorm_kernel<T>, dim3(n_out), dim3(threads), 0, (hipStream_t)stream,   \
                       h, (const T*)delta, w, (T*)out, rows, hidden, eps);                          \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_rmsnorm_##SUF(void* out, const void* x, const float* w, long long rows, int n,  \
                                  float eps, void* stream) {                                        \
    if (rows <= 0) return 0;                                                                        \
    const int wpb = 4;                                                                              \
    hipLaunchKernelGGL(rmsnorm_kernel<T>, dim3((unsigned)((rows + wpb - 1) / wpb)),                 \
                       dim3(wpb * JV_WAVE), 0, (hipStream_t)stream, (T*)out, (const T*)x, w, rows,  \
                       n, eps);                                                                     \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_silu_mul_##SUF(void* out, const void* gu, long long n_tokens, int inter,        \
                                   void* stream) {                                                  \
    const long long total = n_tokens * inter;                                                       \
    if (total <= 0) return 0;                                                                       \
    long long blocks = (total + 255) / 256;                                                         \
    if (blocks > 65536) blocks = 65536;                                                             \
    hipLaunchKernelGGL(silu_mul_kernel<T>, dim3((unsigned)blocks), dim3(256), 0,                    \
                       (hipStream_t)stream, (T*)out, (const T*)gu, total, inter);                   \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_cast_rows_##SUF(void* out, const float* x, const int* rows, int n_out, int n,   \
                                    void* stream) {                                                 \
    if (n_out <= 0) return 0;                                                                       \
    hipLaunchKernelGGL(cast_rows_kernel<T>, dim3(n_out), dim3(256), 0, (hipStream_t)stream,         \
                       (T*)out, x, rows, n);                                                        \
    return JV_LAUNCH_CHECK();                                                                       \
  }

DEFINE_ELEMENTWISE(bf16, bf16_t)
DEFINE_ELEMENTWISE(f32, float)
