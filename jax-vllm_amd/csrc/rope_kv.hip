// Attention input preparation, one launch per layer:
//   per-head RMSNorm of q and k (optional) -> rotary position encoding (optional)
//   -> q written back in place, k and v written into their cache pages.
// Input is the fused projection output qkv[t, (nq + 2*nkv) * D]; head j of q is
// columns [j*D, (j+1)*D), then the k heads, then the v heads.
//
// Rotation (float): for pair index p < rotary_dim/2, angle = pos * inv_freq[p], cosine and sine
// taken from a per-step table;
//   half-split pairing:  (x[p], x[p + rotary_dim/2])     interleaved: (x[2p], x[2p+1])
//   (a, b) -> (a*cos - b*sin, b*cos + a*sin);  elements >= rotary_dim pass through.
// Cache layout: K pages[page][kv_head][slot][D]; V pages[page][kv_head][D][slot] (transposed,
// so that the attention kernels find a page's keys contiguous per d);
// slot_mapping[t] = page * page_size + slot, or a negative value for a token whose k/v must
// not be stored.
#include "common.h"

#define ROPE_MAX_D 512

// cos_sin[t, 0:half] = cos(pos_t * inv_freq), cos_sin[t, half:2*half] = sin(...), all float.
// Computed once per step: every layer of the step rotates by the same angles.
__global__ void rope_table_kernel(float* __restrict__ cos_sin, const int* __restrict__ positions,
                                  const float* __restrict__ inv_freq, int half) {
  const long long t = blockIdx.x;
  const float pos = (float)positions[t];
  for (int p = threadIdx.x; p < half; p += blockDim.x) {
    float s, c;
    sincosf(pos * inv_freq[p], &s, &c);
    cos_sin[t * 2 * half + p] = c;
    cos_sin[t * 2 * half + half + p] = s;
  }
}

extern "C" int jv_rope_table(float* cos_sin, const int* positions, const float* inv_freq,
                             int n_tokens, int half, void* stream) {
  if (n_tokens <= 0 || half <= 0) return 0;
  hipLaunchKernelGGL(rope_table_kernel, dim3(n_tokens), dim3(half >= 128 ? 128 : 64), 0,
                     (hipStream_t)stream, cos_sin, positions, inv_freq, half);
  return JV_LAUNCH_CHECK();
}

// One wave per (token, head); 4 heads per block.
template <typename T>
__global__ void __launch_bounds__(256) qk_norm_rope_write_kernel(
    T* __restrict__ qkv, const int* __restrict__ slot_mapping, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin, int rotary_dim,
    int interleaved, T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nq,
    int nkv, int D) {
  extern __shared__ float lds[];  // [4 waves][D]
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE;
  float* buf = lds + wid * D;
  const long long t = blockIdx.x;
  const int n_heads = nq + 2 * nkv;
  const int head = blockIdx.y * 4 + wid;
  const bool live = head < n_heads;
  T* row = qkv + t * (long long)n_heads * D;
  const long long slot = slot_mapping ? (long long)slot_mapping[t] : -1;
  const bool store = (slot >= 0) && (k_pages != nullptr);
  const long long page = store ? slot / page_size : 0;
  const int off = store ? (int)(slot - page * page_size) : 0;
  const int half = rotary_dim / 2;
  const bool is_v = live && head >= nq + nkv;
  const bool is_q = live && head < nq;
  const bool is_k = live && !is_q && !is_v;
  T* x = row + (long long)(live ? head : 0) * D;
  if (is_v && store) {  // v head: copied to its (transposed) page
    const int kvh = head - nq - nkv;
    T* dst = v_pages + (page * nkv + kvh) * (long long)D * page_size + off;
    for (int d = lane; d < D; d += JV_WAVE) dst[(long long)d * page_size] = x[d];
  }
  const bool work = is_q || (is_k && store);  // a k head that nobody will read is skipped
  const float* w = is_q ? q_w : k_w;
  if (work) {
    float ss = 0.f;
    for (int d = lane; d < D; d += JV_WAVE) {
      const float v = to_f32(x[d]);
      buf[d] = v;
      ss += v * v;
    }
    if (w) {
      ss = wave_sum(ss);
      const float inv = rsqrtf(ss / (float)D + eps);
      for (int d = lane; d < D; d += JV_WAVE) buf[d] = buf[d] * inv * w[d];
    }
  }
  __syncthreads();  // buf written -> readable by the wave's other lanes (every wave arrives once)
  if (work) {
    T* dst = is_q ? x : k_pages + ((page * nkv + (head - nq)) * page_size + off) * (long long)D;
    if (cos_sin) {
      const float* cs = cos_sin + t * rotary_dim;
      for (int p = lane; p < half; p += JV_WAVE) {
        const int ia = interleaved ? 2 * p : p;
        const int ib = interleaved ? 2 * p + 1 : p + half;
        const float c = cs[p], sn = cs[half + p];
        const float a = buf[ia], b = buf[ib];
        dst[ia] = from_f32<T>(a * c - b * sn);
        dst[ib] = from_f32<T>(b * c + a * sn);
      }
      for (int d = rotary_dim + lane; d < D; d += JV_WAVE) dst[d] = from_f32<T>(buf[d]);
    } else {
      for (int d = lane; d < D; d += JV_WAVE) dst[d] = from_f32<T>(buf[d]);
    }
  }
}

// Fast path for head sizes that are a multiple of 64 with half-split pairing and rotary_dim/2 a
// multiple of 64 (D = 128 or 256 fully rotated): lane l holds elements l, l+64, ..., so both
// members of every rotation pair sit in one lane: no LDS, no barrier.  One wave takes
// `heads_per_wave` consecutive heads of one token.
template <typename T, int E, int NP>
__global__ void __launch_bounds__(256) qk_norm_rope_write_fast_kernel(
    T* __restrict__ qkv, const float* __restrict__ parts, long long part_stride,
    const int* __restrict__ slot_mapping, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin, int rotary_dim,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nq, int nkv,
    int heads_per_wave) {
  constexpr int D = E * 64;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const long long t = blockIdx.x;
  const int n_heads = nq + 2 * nkv;
  T* row = qkv + t * (long long)n_heads * D;
  const long long slot = slot_mapping ? (long long)slot_mapping[t] : -1;
  const bool store = (slot >= 0) && (k_pages != nullptr);
  const long long page = store ? slot / page_size : 0;
  const int off = store ? (int)(slot - page * page_size) : 0;
  const int half = rotary_dim / 2, HE = half / 64;   // pair (e, e + HE) for e < HE
  float cs[E], sn[E];                                 // cos/sin of this lane's pair indices
  if (cos_sin) {
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (e < HE) {
        cs[e] = cos_sin[t * rotary_dim + e * 64 + lane];
        sn[e] = cos_sin[t * rotary_dim + half + e * 64 + lane];
      }
  }
  const int h0 = (blockIdx.y * 4 + wid) * heads_per_wave;
  for (int head = h0; head < h0 + heads_per_wave && head < n_heads; ++head) {
    T* x = row + (long long)head * D;
    float v[E], wv[E];
    if (NP == 0) {
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] = to_f32(x[e * 64 + lane]);
    } else {
      // the projection comes as NP float partial products [NP][tokens][heads * D] of a matrix
      // product whose inner size was shared out: all are asked for at once and added in order
      const float* px = parts + (t * n_heads + head) * (long long)D + lane;
      float pv[NP > 0 ? NP : 1][E];
#pragma unroll
      for (int q = 0; q < NP; ++q)
#pragma unroll
        for (int e = 0; e < E; ++e) pv[q][e] = px[q * part_stride + e * 64];
#pragma unroll
      for (int e = 0; e < E; ++e) {
        v[e] = pv[0][e];
#pragma unroll
        for (int q = 1; q < NP; ++q) v[e] += pv[q][e];
      }
    }
    {  // the norm weights are asked for together with the head, not after its reduction
      const float* w0 = head < nq ? q_w : (head < nq + nkv ? k_w : nullptr);
#pragma unroll
      for (int e = 0; e < E; ++e) wv[e] = w0 ? w0[e * 64 + lane] : 1.f;
    }
    if (head >= nq + nkv) {  // v head: copied to its (transposed) page
      if (store) {
        T* dst = v_pages + (page * nkv + (head - nq - nkv)) * (long long)D * page_size + off;
#pragma unroll
        for (int e = 0; e < E; ++e) dst[(long long)(e * 64 + lane) * page_size] = from_f32<T>(v[e]);
      }
      continue;
    }
    const bool is_q = head < nq;
    if (!is_q && !store) continue;
    const float* w = is_q ? q_w : k_w;
    if (w) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < E; ++e) ss += v[e] * v[e];
      ss = wave_sum(ss);
      const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
      for (int e = 0; e < E; ++e) v[e] = v[e] * inv * wv[e];
    }
    if (cos_sin) {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (e < HE) {
          const float a = v[e], b = v[e + HE];
          v[e] = a * cs[e] - b * sn[e];
          v[e + HE] = b * cs[e] + a * sn[e];
        }
    }
    T* dst = is_q ? x : k_pages + ((page * nkv + (head - nq)) * page_size + off) * (long long)D;
#pragma unroll
    for (int e = 0; e < E; ++e) dst[e * 64 + lane] = from_f32<T>(v[e]);
  }
}

#define DEFINE_ROPE(SUF, T)                                                                        \
  extern "C" int jv_qk_norm_rope_write_##SUF(                                                      \
      void* qkv, const int* slot_mapping, const float* q_w, const float* k_w, float eps,           \
      const float* cos_sin, int rotary_dim, int interleaved, void* k_pages, void* v_pages,         \
      int page_size, int n_tokens, int nq, int nkv, int D, void* stream) {                         \
    if (n_tokens <= 0) return 0;                                                                   \
    if (D > ROPE_MAX_D || rotary_dim > D || (rotary_dim & 1)) return (int)hipErrorInvalidValue;    \
    const int n_heads = nq + 2 * nkv;                                                              \
    if ((n_heads + 3) / 4 > 65535) return (int)hipErrorInvalidValue;                               \
    const int half = rotary_dim / 2;                                                               \
    if ((D == 128 || D == 256) && !interleaved && (!cos_sin || (half % 64 == 0 && half > 0))) {    \
      /* many tokens: a wave walks several heads; few tokens: one head per wave for parallelism */ \
      const int hpw = n_tokens >= 256 ? (n_heads + 3) / 4 : 1;                                     \
      const int gy = (n_heads + 4 * hpw - 1) / (4 * hpw);                                          \
      if (D == 128)                                                                                \
        hipLaunchKernelGGL((qk_norm_rope_write_fast_kernel<T, 2, 0>), dim3(n_tokens, gy),          \
                           dim3(256), 0, (hipStream_t)stream, (T*)qkv, (const float*)nullptr, 0ll, \
                           slot_mapping, q_w, k_w, eps, cos_sin, rotary_dim, (T*)k_pages,          \
                           (T*)v_pages, page_size, nq, nkv, hpw);                                  \
      else                                                                                         \
        hipLaunchKernelGGL((qk_norm_rope_write_fast_kernel<T, 4, 0>), dim3(n_tokens, gy),          \
                           dim3(256), 0, (hipStream_t)stream, (T*)qkv, (const float*)nullptr, 0ll, \
                           slot_mapping, q_w, k_w, eps, cos_sin, rotary_dim, (T*)k_pages,          \
                           (T*)v_pages, page_size, nq, nkv, hpw);                                  \
      return JV_LAUNCH_CHECK();                                                                    \
    }                                                                                              \
    hipLaunchKernelGGL(qk_norm_rope_write_kernel<T>, dim3(n_tokens, (n_heads + 3) / 4), dim3(256), \
                       4 * D * sizeof(float), (hipStream_t)stream, (T*)qkv, slot_mapping, q_w,     \
                       k_w, eps, cos_sin, rotary_dim, interleaved, (T*)k_pages, (T*)v_pages,       \
                       page_size, nq, nkv, D);                                                     \
    return JV_LAUNCH_CHECK();                                                                      \
  }

DEFINE_ROPE(bf16, bf16_t)
DEFINE_ROPE(f32, float)

// The same with the projection given as n_parts (2..4) float partial products
// [n_parts][tokens][heads * D]; q is written to `qkv` (the q heads of each row), k and v to their
// pages.  Only what the fast path takes: head size 128 or 256, half-split pairing, fully rotated
// or not rotated; anything else is refused (the caller then asks for a whole product).
template <typename T, int E, int NP>
static int launch_rope_parts(void* qkv, const float* parts, long long part_stride, const int* slot_mapping,
                             const float* q_w, const float* k_w, float eps, const float* cos_sin, int rotary_dim,
                             void* k_pages, void* v_pages, int page_size, int n_tokens, int nq, int nkv,
                             void* stream) {
  const int n_heads = nq + 2 * nkv;
  const int hpw = n_tokens >= 256 ? (n_heads + 3) / 4 : 1;
  const int gy = (n_heads + 4 * hpw - 1) / (4 * hpw);
  hipLaunchKernelGGL((qk_norm_rope_write_fast_kernel<T, E, NP>), dim3(n_tokens, gy), dim3(256), 0,
                     (hipStream_t)stream, (T*)qkv, parts, part_stride, slot_mapping, q_w, k_w, eps, cos_sin,
                     rotary_dim, (T*)k_pages, (T*)v_pages, page_size, nq, nkv, hpw);
  return JV_LAUNCH_CHECK();
}

extern "C" int jv_qk_norm_rope_write_parts_bf16(
    void* qkv, const float* parts, int n_parts, long long part_stride, const int* slot_mapping, const float* q_w,
    const float* k_w, float eps, const float* cos_sin, int rotary_dim, void* k_pages, void* v_pages,
    int page_size, int n_tokens, int nq, int nkv, int D, void* stream) {
  if (n_tokens <= 0) return 0;
  const int half = rotary_dim / 2;
  if ((D != 128 && D != 256) || n_parts < 2 || n_parts > 4 || (rotary_dim & 1) || rotary_dim > D ||
      (cos_sin && (half % 64 != 0 || half <= 0)))
    return (int)hipErrorInvalidValue;
#define ROPE_PARTS_CASE(E, NP)                                                                             \
  if (D == 64 * E && n_parts == NP)                                                                        \
    return launch_rope_parts<bf16_t, E, NP>(qkv, parts, part_stride, slot_mapping, q_w, k_w, eps, cos_sin, \
                                            rotary_dim, k_pages, v_pages, page_size, n_tokens, nq, nkv, stream);
  ROPE_PARTS_CASE(2, 2) ROPE_PARTS_CASE(2, 3) ROPE_PARTS_CASE(2, 4)
  ROPE_PARTS_CASE(4, 2) ROPE_PARTS_CASE(4, 3) ROPE_PARTS_CASE(4, 4)
#undef ROPE_PARTS_CASE
  return (int)hipErrorInvalidValue;
}
