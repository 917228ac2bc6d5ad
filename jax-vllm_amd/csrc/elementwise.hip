// Embedding gather, fused residual-add + RMSNorm, plain RMSNorm, SiLU-mul.
// The residual stream is float in every mode; normalised outputs are in the
// activation type T.  All reductions are float.
#include "common.h"

// ---------------------------------------------------------------- embedding gather
// h[t, :] = float(table[ids[t], :]).  One block per token.  An id outside [0, rows) reads nothing:
// its row of h becomes NaN (ids may come straight from a sampling kernel on the device, which answers
// `rows` for a row of logits without a maximum; the host reports that row when it sees the id).
template <typename T>
__global__ void embedding_kernel(float* __restrict__ h, const T* __restrict__ table,
                                 const int* __restrict__ ids, int hidden, int rows) {
  const long long t = blockIdx.x;
  const int id = ids[t];
  const bool inside = id >= 0 && id < rows;
  const T* row = table + (long long)(inside ? id : 0) * hidden;
  float* out = h + t * hidden;
  const float nan = __builtin_nanf("");
  // 16 bytes of the table a lane where the row allows it (a width that is a multiple of the pieces'
  // elements keeps every row of table and of h aligned), element by element otherwise
  constexpr int V = 16 / sizeof(T);
  if (hidden % V == 0) {
    typedef T tv __attribute__((ext_vector_type(V)));
    typedef float f4 __attribute__((ext_vector_type(4)));
    for (int i = threadIdx.x * V; i < hidden; i += blockDim.x * V) {
      const tv v = *(const tv*)(row + i);
#pragma unroll
      for (int j = 0; j < V; j += 4) {
        f4 o;
#pragma unroll
        for (int e = 0; e < 4; ++e) o[e] = inside ? to_f32(v[j + e]) : nan;
        *(f4*)(out + i + j) = o;
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
      const float v = to_f32(row[i]);
      out[i] = inside ? v : nan;
    }
  }
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

// The same for widths that are a multiple of 4 and at most 4 * 8 * blockDim: 16-byte loads of
// the residual stream, the row kept in registers between the two passes.
template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float4 type; };
template <> struct Vec4<bf16_t> { typedef __attribute__((ext_vector_type(4))) __bf16 type; };

template <typename T>
__device__ __forceinline__ float4 load4(const T* p) {
  typename Vec4<T>::type v = *(const typename Vec4<T>::type*)p;
  return float4{to_f32<T>(v[0]), to_f32<T>(v[1]), to_f32<T>(v[2]), to_f32<T>(v[3])};
}
template <>
__device__ __forceinline__ float4 load4<float>(const float* p) { return *(const float4*)p; }

template <typename T>
__device__ __forceinline__ void store4(T* p, float4 v) {
  typename Vec4<T>::type o;
  o[0] = from_f32<T>(v.x); o[1] = from_f32<T>(v.y); o[2] = from_f32<T>(v.z); o[3] = from_f32<T>(v.w);
  *(typename Vec4<T>::type*)p = o;
}
template <>
__device__ __forceinline__ void store4<float>(float* p, float4 v) { *(float4*)p = v; }

// eight neighbours as floats: one 16-byte load of bfloat16, two of float
template <typename T>
__device__ __forceinline__ void load8(const T* p, float (&v)[8]) {
  typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
  const bf16x8_t x = *(const bf16x8_t*)p;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (float)x[e];
}
template <>
__device__ __forceinline__ void load8<float>(const float* p, float (&v)[8]) {
  const float4 a = *(const float4*)p, b = *(const float4*)(p + 4);
  v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}

#define ARN_MAX_V 8
#define ARN_MAX_PARTS 4
// V = 16-byte pieces of the residual row per thread (the launch picks the least that covers the row).  Every
// load (residual, delta, norm weight) is issued before the reduction and none sits inside a branch: a
// piece beyond the row reads the row's last piece again and only its stores and its share of the sum are
// left out (a load inside a branch makes the compiler wait for all loads in flight where the branch
// ends: 1.1 us of a 4.4 us kernel).  A short row's time is the sum of its dependent memory round trips.
template <typename T, int V>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(float* __restrict__ h, const T* __restrict__ delta,
                       const float* __restrict__ w, T* __restrict__ out,
                       const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float red[32];
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  float* hr = h + r * hidden;
  const T* dr = delta ? delta + r * hidden : (const T*)w;      // any readable address: its values get no weight
  T* o = out + i * hidden;
  const int nvec = hidden >> 2;
  float4 x[V], ww[V], d[V];
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const int c = min((int)(threadIdx.x + k * blockDim.x), nvec - 1);
    ww[k] = *(const float4*)(w + 4 * c);
    x[k] = *(const float4*)(hr + 4 * c);
    d[k] = load4<T>(dr + (delta ? 4 * c : 0));
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    float4 v = x[k];
    if (delta) { v.x += d[k].x; v.y += d[k].y; v.z += d[k].z; v.w += d[k].w; }
    if (c < nvec) {
      if (delta && !rows) *(float4*)(hr + 4 * c) = v;
      ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    x[k] = v;
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const int c = threadIdx.x + k * blockDim.x;
    const float4 v = x[k];
    if (c < nvec)
      store4<T>(o + 4 * c, float4{v.x * inv * ww[k].x, v.y * inv * ww[k].y, v.z * inv * ww[k].z, v.w * inv * ww[k].w});
  }
}

// The same with the delta given as NP float partial products of a matrix product whose inner
// size was shared out to NP blocks: parts[q][r][:], added first, in the order of q, then to the
// residual.
// EXACT: blocks of 256 threads whose V pieces cover the row exactly (no index is clamped or tested).
template <typename T, int NP, int V, bool EXACT>
__global__ void __launch_bounds__(256)
add_rmsnorm_parts_kernel(float* __restrict__ h, const float* __restrict__ parts, long long part_stride,
                         const float* __restrict__ w, T* __restrict__ out, const int* __restrict__ rows,
                         int hidden, float eps) {
  __shared__ float red[32];
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  float* hr = h + r * hidden;
  const float* pr = parts + r * hidden;
  T* o = out + i * hidden;
  const int nvec = EXACT ? V * 256 : hidden >> 2;
  const int nthreads = EXACT ? 256 : blockDim.x;
  float4 x[V], ww[V], e[V][NP];
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const int c = EXACT ? (int)threadIdx.x + k * 256 : min((int)(threadIdx.x + k * nthreads), nvec - 1);
    ww[k] = *(const float4*)(w + 4 * c);
    x[k] = *(const float4*)(hr + 4 * c);
#pragma unroll
    for (int q = 0; q < NP; ++q) e[k][q] = *(const float4*)(pr + q * part_stride + 4 * c);
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const int c = threadIdx.x + k * nthreads;
    float4 d = e[k][0];
#pragma unroll
    for (int q = 1; q < NP; ++q) { d.x += e[k][q].x; d.y += e[k][q].y; d.z += e[k][q].z; d.w += e[k][q].w; }
    float4 v = x[k];
    v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
    if (EXACT || c < nvec) {
      if (!rows) *(float4*)(hr + 4 * c) = v;
      ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
    }
    x[k] = v;
  }
  ss = block_sum(ss, red);
  const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
  for (int k = 0; k < V; ++k) {
    const int c = threadIdx.x + k * nthreads;
    const float4 v = x[k];
    if (EXACT || c < nvec)
      store4<T>(o + 4 * c, float4{v.x * inv * ww[k].x, v.y * inv * ww[k].y, v.z * inv * ww[k].z, v.w * inv * ww[k].w});
  }
}

// The residual step of a row shared out to hidden / 512 blocks, with the norm's scale left to the reader:
//   h[r] += parts[0][r] + parts[1][r] + ... (in that order), xg[r] = T(h[r] * w) (NOT normalised),
//   ssq[r][b] = sum of squares of block b's 512 columns of the new h[r] (rows of 16 floats, hidden / 512 <= 16 of
//   them written).
// A matrix product that takes xg multiplies its output rows by rsqrt(sum_b ssq[r][b] / hidden + eps)
// (the scale of a row commutes with the product).  One compute unit no longer has to pull a whole
// row's five arrays: 2.3 us after a product against 3.9 for the norm kernel at 8 rows of 4,096.
#define ARN_SHARE 512
template <typename T, int NP>
__global__ void __launch_bounds__(128)
add_parts_unscaled_kernel(float* __restrict__ h, const float* __restrict__ parts, long long part_stride,
                          const float* __restrict__ w, T* __restrict__ xg, float* __restrict__ ssq, int hidden) {
  __shared__ float red[2];
  const long long r = blockIdx.y;
  const int c = blockIdx.x * (ARN_SHARE / 4) + threadIdx.x;      // 16-byte piece of the row
  float* hr = h + r * hidden;
  const float* pr = parts + r * hidden;
  const float4 ww = *(const float4*)(w + 4 * c);
  float4 v = *(const float4*)(hr + 4 * c), e[NP];
#pragma unroll
  for (int q = 0; q < NP; ++q) e[q] = *(const float4*)(pr + q * part_stride + 4 * c);
  float4 d = e[0];
#pragma unroll
  for (int q = 1; q < NP; ++q) { d.x += e[q].x; d.y += e[q].y; d.z += e[q].z; d.w += e[q].w; }
  v.x += d.x; v.y += d.y; v.z += d.z; v.w += d.w;
  *(float4*)(hr + 4 * c) = v;
  store4<T>(xg + r * hidden + 4 * c, float4{v.x * ww.x, v.y * ww.y, v.z * ww.z, v.w * ww.w});
  const float s = wave_sum(v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) ssq[r * 16 + blockIdx.x] = red[0] + red[1];       // rows of 16 shares, gridDim.x of them written
}

// threads of a block and 16-byte pieces per thread for a row of nvec pieces (nvec <= 8 * 256)
static void arn_shape(int nvec, int* threads, int* v) {
  *threads = nvec >= 1024 ? 256 : (nvec >= 256 ? 128 : 64);
  const int need = (nvec + *threads - 1) / *threads;
  *v = need <= 1 ? 1 : need <= 2 ? 2 : need <= 4 ? 4 : need <= 5 ? 5 : 8;
}
template <typename T>
static void launch_arn_vec(int v, int n_out, int threads, hipStream_t st, float* h, const T* delta, const float* w, T* out,
                           const int* rows, int hidden, float eps) {
#define ARN_GO(V) hipLaunchKernelGGL((add_rmsnorm_vec_kernel<T, V>), dim3(n_out), dim3(threads), 0, st, h, delta, w, out, rows, hidden, eps)
  switch (v) {
    case 1: ARN_GO(1); break;
    case 2: ARN_GO(2); break;
    case 4: ARN_GO(4); break;
    case 5: ARN_GO(5); break;
    default: ARN_GO(8); break;
  }
#undef ARN_GO
}
template <typename T, int NP>
static void launch_arn_parts(int v, int n_out, int threads, hipStream_t st, float* h, const float* parts, long long part_stride,
                             const float* w, T* out, const int* rows, int hidden, float eps) {
#define ARN_GO(V)                                                                                                \
  if (threads == 256 && hidden == 4 * 256 * V)                                                                   \
    hipLaunchKernelGGL((add_rmsnorm_parts_kernel<T, NP, V, true>), dim3(n_out), dim3(256), 0, st, h, parts,       \
                       part_stride, w, out, rows, hidden, eps);                                                  \
  else                                                                                                           \
    hipLaunchKernelGGL((add_rmsnorm_parts_kernel<T, NP, V, false>), dim3(n_out), dim3(threads), 0, st, h, parts,  \
                       part_stride, w, out, rows, hidden, eps)
  switch (v) {
    case 1: ARN_GO(1); break;
    case 2: ARN_GO(2); break;
    case 4: ARN_GO(4); break;
    case 5: ARN_GO(5); break;
    default: ARN_GO(8); break;
  }
#undef ARN_GO
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

// ---------------------------------------------------------------- gate activation times up
// out[t, j] = act(gate) * up in float, act one of JV_ACT_*.  Two layouts of gu[t, 2*inter]:
// halves (gate = gu[t, j], up = gu[t, inter + j]) or interleaved (gate = gu[t, 2j], up = gu[t, 2j+1]).
// Interleaved layout (gate and up alternate along the row): out[t, j] = act(gu[t, 2j]) * gu[t, 2j+1];
// each thread takes four outputs (8 inputs, 16 bytes of bfloat16) when inter % 4 == 0.
template <typename T, int ACT>
__global__ void gated_mul_pairs_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter) {
  const long long t = blockIdx.y;
  const int j = (blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (j >= inter) return;
  const T* gp = gu + t * 2 * inter + 2 * j;
  T* op = out + t * inter + j;
  if ((inter & 3) == 0) {
    float v[8];
    load8<T>(gp, v);
    store4<T>(op, float4{jv_gated(ACT, v[0], v[1]), jv_gated(ACT, v[2], v[3]), jv_gated(ACT, v[4], v[5]),
                         jv_gated(ACT, v[6], v[7])});
  } else {
    for (int e = 0; e < 4 && j + e < inter; ++e)
      op[e] = from_f32<T>(jv_gated(ACT, to_f32(gp[2 * e]), to_f32(gp[2 * e + 1])));
  }
}

// grid (column blocks, tokens); each thread takes 4 neighbouring columns when inter % 4 == 0.
template <typename T, int VEC, int ACT>
__global__ void gated_mul_kernel(T* __restrict__ out, const T* __restrict__ gu, int inter) {
  const long long t = blockIdx.y;
  const int j = (blockIdx.x * blockDim.x + threadIdx.x) * VEC;
  if (j >= inter) return;
  const T* gp = gu + t * 2 * inter + j;
  T* op = out + t * inter + j;
  if (VEC == 4) {
    const float4 g = load4<T>(gp), u = load4<T>(gp + inter);
    store4<T>(op, float4{jv_gated(ACT, g.x, u.x), jv_gated(ACT, g.y, u.y), jv_gated(ACT, g.z, u.z),
                         jv_gated(ACT, g.w, u.w)});
  } else {
    op[0] = from_f32<T>(jv_gated(ACT, to_f32(gp[0]), to_f32(gp[inter])));
  }
}

template <typename T, int ACT>
static void launch_gated_mul(T* o, const T* g, unsigned ny, int inter, int interleaved, hipStream_t stream) {
  if (interleaved)
    hipLaunchKernelGGL((gated_mul_pairs_kernel<T, ACT>), dim3(((inter + 3) / 4 + 255) / 256, ny), dim3(256), 0, stream,
                       o, g, inter);
  else if (inter % 4 == 0)
    hipLaunchKernelGGL((gated_mul_kernel<T, 4, ACT>), dim3((inter / 4 + 255) / 256, ny), dim3(256), 0, stream, o, g,
                       inter);
  else
    hipLaunchKernelGGL((gated_mul_kernel<T, 1, ACT>), dim3((inter + 255) / 256, ny), dim3(256), 0, stream, o, g,
                       inter);
}

// ---------------------------------------------------------------- float -> T copy of selected rows
template <typename T>
__global__ void cast_rows_kernel(T* __restrict__ out, const float* __restrict__ x,
                                 const int* __restrict__ rows, int n) {
  const long long i = blockIdx.x;
  const long long r = rows ? (long long)rows[i] : i;
  for (int c = threadIdx.x; c < n; c += blockDim.x) out[i * n + c] = from_f32<T>(x[r * n + c]);
}

// ---------------------------------------------------------------- bias of a projection
// y[r, c] += bias[c], summed in float; grid (column blocks, rows)
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, int n) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= n) return;
  T* at = y + (long long)blockIdx.y * n + c;
  *at = from_f32<T>(to_f32(*at) + bias[c]);
}

#define DEFINE_ELEMENTWISE(SUF, T)                                                                  \
  extern "C" int jv_embedding_##SUF(float* h, const void* table, const int* ids, int n_tokens,      \
                                    int hidden, int rows, void* stream) {                           \
    if (n_tokens <= 0) return 0;                                                                    \
    hipLaunchKernelGGL(embedding_kernel<T>, dim3(n_tokens), dim3(256), 0, (hipStream_t)stream, h,   \
                       (const T*)table, ids, hidden, rows);                                         \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_add_rmsnorm_##SUF(float* h, const void* delta, const float* w, void* out,       \
                                      const int* rows, int n_out, int hidden, float eps,            \
                                      void* stream) {                                               \
    if (n_out <= 0) return 0;                                                                       \
    const int threads = hidden >= 2048 ? 512 : 256;                                                 \
    if (hidden % 4 == 0 && hidden <= 4 * ARN_MAX_V * 256) {                                         \
      int vt, v;                                                                                    \
      arn_shape(hidden / 4, &vt, &v);                                                               \
      launch_arn_vec<T>(v, n_out, vt, (hipStream_t)stream, h, (const T*)delta, w, (T*)out, rows,    \
                        hidden, eps);                                                               \
    } else {                                                                                        \
      hipLaunchKernelGGL(add_rmsnorm_kernel<T>, dim3(n_out), dim3(threads), 0, (hipStream_t)stream, \
                         h, (const T*)delta, w, (T*)out, rows, hidden, eps);                        \
    }                                                                                               \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  /* the delta as n_parts float partial products [n_parts][rows of h][hidden], added in order */   \
  extern "C" int jv_add_rmsnorm_parts_##SUF(float* h, const float* parts, int n_parts,              \
                                            long long part_stride, const float* w, void* out,       \
                                            const int* rows, int n_out, int hidden, float eps,      \
                                            void* stream) {                                         \
    if (n_out <= 0) return 0;                                                                       \
    if (n_parts < 1 || n_parts > ARN_MAX_PARTS || hidden % 4 != 0 || hidden > 4 * ARN_MAX_V * 256)  \
      return (int)hipErrorInvalidValue;                                                             \
    int vt, v;                                                                                      \
    arn_shape(hidden / 4, &vt, &v);                                                                 \
    hipStream_t st = (hipStream_t)stream;                                                           \
    switch (n_parts) {                                                                              \
      case 1: launch_arn_parts<T, 1>(v, n_out, vt, st, h, parts, part_stride, w, (T*)out, rows, hidden, eps); break; \
      case 2: launch_arn_parts<T, 2>(v, n_out, vt, st, h, parts, part_stride, w, (T*)out, rows, hidden, eps); break; \
      case 3: launch_arn_parts<T, 3>(v, n_out, vt, st, h, parts, part_stride, w, (T*)out, rows, hidden, eps); break; \
      default: launch_arn_parts<T, 4>(v, n_out, vt, st, h, parts, part_stride, w, (T*)out, rows, hidden, eps); break; \
    }                                                                                               \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  /* the same residual step with the norm's scale left to the reader: see add_parts_unscaled_kernel; */ \
  /* ssq must hold n_rows * 16 floats */                                                            \
  extern "C" int jv_add_parts_unscaled_##SUF(float* h, const float* parts, int n_parts,             \
                                             long long part_stride, const float* w, void* xg,       \
                                             float* ssq, int n_rows, int hidden, void* stream) {    \
    if (n_rows <= 0) return 0;                                                                      \
    if (n_parts < 1 || n_parts > ARN_MAX_PARTS || hidden % ARN_SHARE != 0 || n_rows > 65535 ||      \
        hidden / ARN_SHARE > 16)                                                                    \
      return (int)hipErrorInvalidValue;                                                             \
    const dim3 grid(hidden / ARN_SHARE, n_rows);                                                    \
    hipStream_t st = (hipStream_t)stream;                                                           \
    switch (n_parts) {                                                                              \
      case 1: hipLaunchKernelGGL((add_parts_unscaled_kernel<T, 1>), grid, dim3(128), 0, st, h, parts, part_stride, w, (T*)xg, ssq, hidden); break; \
      case 2: hipLaunchKernelGGL((add_parts_unscaled_kernel<T, 2>), grid, dim3(128), 0, st, h, parts, part_stride, w, (T*)xg, ssq, hidden); break; \
      case 3: hipLaunchKernelGGL((add_parts_unscaled_kernel<T, 3>), grid, dim3(128), 0, st, h, parts, part_stride, w, (T*)xg, ssq, hidden); break; \
      default: hipLaunchKernelGGL((add_parts_unscaled_kernel<T, 4>), grid, dim3(128), 0, st, h, parts, part_stride, w, (T*)xg, ssq, hidden); break; \
    }                                                                                               \
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
  extern "C" int jv_gated_mul_##SUF(void* out, const void* gu, long long n_tokens, int inter,       \
                                    int interleaved, int act, void* stream) {                      \
    if (n_tokens <= 0 || inter <= 0) return 0;                                                      \
    if (!jv_act_known(act)) return (int)hipErrorInvalidValue;                                       \
    for (long long t0 = 0; t0 < n_tokens; t0 += 65535) { /* grid.y limit */                         \
      const unsigned ny = (unsigned)(n_tokens - t0 < 65535 ? n_tokens - t0 : 65535);                \
      T* o = (T*)out + t0 * inter;                                                                  \
      const T* g = (const T*)gu + t0 * 2 * inter;                                                   \
      if (act == JV_ACT_GELU_TANH)                                                                  \
        launch_gated_mul<T, JV_ACT_GELU_TANH>(o, g, ny, inter, interleaved, (hipStream_t)stream);   \
      else                                                                                          \
        launch_gated_mul<T, JV_ACT_SILU>(o, g, ny, inter, interleaved, (hipStream_t)stream);        \
    }                                                                                               \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_cast_rows_##SUF(void* out, const float* x, const int* rows, int n_out, int n,   \
                                    void* stream) {                                                 \
    if (n_out <= 0) return 0;                                                                       \
    hipLaunchKernelGGL(cast_rows_kernel<T>, dim3(n_out), dim3(256), 0, (hipStream_t)stream,         \
                       (T*)out, x, rows, n);                                                        \
    return JV_LAUNCH_CHECK();                                                                       \
  }                                                                                                 \
  extern "C" int jv_add_bias_##SUF(void* y, const float* bias, long long rows, int n, void* stream) { \
    if (rows <= 0 || n <= 0) return 0;                                                              \
    for (long long r0 = 0; r0 < rows; r0 += 65535) { /* grid.y limit */                             \
      const unsigned ny = (unsigned)(rows - r0 < 65535 ? rows - r0 : 65535);                        \
      hipLaunchKernelGGL(add_bias_kernel<T>, dim3((n + 255) / 256, ny), dim3(256), 0,               \
                         (hipStream_t)stream, (T*)y + r0 * n, bias, n);                             \
    }                                                                                               \
    return JV_LAUNCH_CHECK();                                                                       \
  }

DEFINE_ELEMENTWISE(bf16, bf16_t)
DEFINE_ELEMENTWISE(f32, float)
