// Paged causal attention, generic path: any head size up to 512, any head counts,
// any page size, float or bf16 storage, all arithmetic in float.  It is the kernel
// of the 32-bit path and the fallback of the bf16 path for shapes the MFMA kernel
// refuses.  One 64-lane block per (token, q head); keys are walked in tiles of 64
// with a running (max, sum) softmax.
//
//   query token t of request r = token_req[t] sits at absolute position p = positions[t]
//   and sees keys j with  max(0, p - window + 1) <= j <= p   (window <= 0: all j <= p);
//   key j lives in page block_tables[r, j / page_size] at slot j % page_size;
//   q head h reads kv head h / (nq / nkv).
// Cache layout: K pages[page][kv_head][slot][D], V pages[page][kv_head][D][slot].
#include "common.h"

#define GEN_MAX_E 8  // head size up to 64 * 8

template <typename T>
__global__ void __launch_bounds__(64)
paged_attention_generic_kernel(T* __restrict__ out, const T* __restrict__ q, long long q_row_stride,
                               const T* __restrict__ k_pages, const T* __restrict__ v_pages,
                               const int* __restrict__ block_tables, int table_stride,
                               const int* __restrict__ token_req, const int* __restrict__ positions,
                               int page_size, int nq, int nkv, int D, float scale, int window) {
  extern __shared__ float lds[];      // q[D] | p[64] | V offsets of the tile's keys as long long [64]
  float* qs = lds;
  float* ps = lds + D;
  long long* offs = (long long*)(ps + 64 + ((D & 1) ? 1 : 0));
  const int lane = threadIdx.x;
  const long long t = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / (nq / nkv);
  const int r = token_req[t];
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* table = block_tables + (long long)r * table_stride;
  const T* qv = q + t * q_row_stride + (long long)h * D;
  for (int d = lane; d < D; d += 64) qs[d] = to_f32(qv[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[GEN_MAX_E];
#pragma unroll
  for (int e = 0; e < GEN_MAX_E; ++e) acc[e] = 0.f;

  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    long long off = 0;
    if (valid) {
      const long long page = table[j / page_size];
      const T* kr = k_pages + ((page * nkv + kvh) * page_size + (j % page_size)) * (long long)D;
      off = (page * nkv + kvh) * (long long)D * page_size + (j % page_size);
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * to_f32(kr[d]);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: key j0 is always valid
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);        // m = -inf on the first tile gives 0
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();  // previous tile's readers are done with ps / offs
    ps[lane] = p;
    offs[lane] = off;
    __syncthreads();
    const int n = (pos - j0 + 1 < 64) ? pos - j0 + 1 : 64;
#pragma unroll
    for (int e = 0; e < GEN_MAX_E; ++e) {
      const int d = lane + 64 * e;
      if (d < D) {
        float a = acc[e] * alpha;
        for (int jj = 0; jj < n; ++jj) a += ps[jj] * to_f32(v_pages[offs[jj] + (long long)d * page_size]);
        acc[e] = a;
      }
    }
  }
  const float inv_l = 1.f / l;
  T* o = out + t * (long long)nq * D + (long long)h * D;
#pragma unroll
  for (int e = 0; e < GEN_MAX_E; ++e) {
    const int d = lane + 64 * e;
    if (d < D) o[d] = from_f32<T>(acc[e] * inv_l);
  }
}

#define DEFINE_ATTN_GENERIC(SUF, T)                                                                \
  extern "C" int jv_paged_attention_generic_##SUF(                                                 \
      void* out, const void* q, long long q_row_stride, const void* k_pages, const void* v_pages,  \
      const int* block_tables, int table_stride, const int* token_req, const int* positions,       \
      int page_size, int n_tokens, int nq, int nkv, int D, float scale, int window,                \
      void* stream) {                                                                              \
    if (n_tokens <= 0) return 0;                                                                   \
    if (D > 64 * GEN_MAX_E || nkv <= 0 || nq % nkv != 0 || page_size <= 0)                         \
      return (int)hipErrorInvalidValue;                                                            \
    const size_t shmem = (D + 64 + 2) * sizeof(float) + 64 * sizeof(long long);                    \
    hipLaunchKernelGGL(paged_attention_generic_kernel<T>, dim3(n_tokens, nq), dim3(64), shmem,     \
                       (hipStream_t)stream, (T*)out, (const T*)q, q_row_stride,                    \
                       (const T*)k_pages, (const T*)v_pages, block_tables, table_stride,           \
                       token_req, positions, page_size, nq, nkv, D, scale, window);                \
    return JV_LAUNCH_CHECK();                                                                      \
  }

DEFINE_ATTN_GENERIC(bf16, bf16_t)
DEFINE_ATTN_GENERIC(f32, float)
