// Attention input preparation, one launch per layer:
//   per-head RMSNorm of q and k (optional) -> rotary position encoding (optional)
//   -> q written back in place, k and v written into their cache pages.
// Input is the fused projection output qkv[t, (nq + 2*nkv) * D]; head j of q is
// columns [j*D, (j+1)*D), then the k heads, then the v heads.
//
// Rotation (float): for pair index p < rotary_dim/2, angle = pos * inv_freq[p];
//   half-split pairing:  (x[p], x[p + rotary_dim/2])     interleaved: (x[2p], x[2p+1])
//   (a, b) -> (a*cos - b*sin, b*cos + a*sin);  elements >= rotary_dim pass through.
// Cache layout: K pages[page][kv_head][slot][D]; V pages[page][kv_head][D][slot] (transposed,
// so that the attention kernels find a page's keys contiguous per d);
// slot_mapping[t] = page * page_size + slot, or a negative value for a token whose k/v must
// not be stored.
#include "common.h"

#define ROPE_MAX_D 512

template <typename T>
__global__ void qk_norm_rope_write_kernel(
    T* __restrict__ qkv, const int* __restrict__ positions, const int* __restrict__ slot_mapping,
    const float* __restrict__ q_w, const float* __restrict__ k_w, float eps,
    const float* __restrict__ inv_freq, int rotary_dim, int interleaved, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int page_size, int nq, int nkv, int D) {
  extern __shared__ float lds[];  // [waves][D]
  const int lane = threadIdx.x & (JV_WAVE - 1), wid = threadIdx.x / JV_WAVE;
  const int nwaves = blockDim.x / JV_WAVE;
  float* buf = lds + wid * D;
  const long long t = blockIdx.x;
  const int n_heads = nq + 2 * nkv;
  T* row = qkv + t * (long long)n_heads * D;
  const float pos = (float)positions[t];
  const long long slot = slot_mapping ? (long long)slot_mapping[t] : -1;
  const bool store = (slot >= 0) && (k_pages != nullptr);
  const long long page = store ? slot / page_size : 0;
  const int off = store ? (int)(slot - page * page_size) : 0;
  const int half = rotary_dim / 2;

  // Every wave runs the same number of rounds so that the block barriers line up.
  for (int base = 0; base < n_heads; base += nwaves) {
    const int head = base + wid;
    const bool live = head < n_heads;
    const bool is_v = live && head >= nq + nkv;
    const bool is_q = live && head < nq;
    const bool is_k = live && !is_q && !is_v;
    T* x = row + (long long)(live ? head : 0) * D;
    if (is_v && store) {  // v head: copy to its page
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
    __syncthreads();  // buf written -> readable by the wave's other lanes
    if (work) {
      T* dst = is_q ? x
                    : k_pages + ((page * nkv + (head - nq)) * page_size + off) * (long long)D;
      if (inv_freq) {
        for (int p = lane; p < half; p += JV_WAVE) {
          const int ia = interleaved ? 2 * p : p;
          const int ib = interleaved ? 2 * p + 1 : p + half;
          float s, c;
          sincosf(pos * inv_freq[p], &s, &c);
          const float a = buf[ia], b = buf[ib];
          dst[ia] = from_f32<T>(a * c - b * s);
          dst[ib] = from_f32<T>(b * c + a * s);
        }
        for (int d = rotary_dim + lane; d < D; d += JV_WAVE) dst[d] = from_f32<T>(buf[d]);
      } else {
        for (int d = lane; d < D; d += JV_WAVE) dst[d] = from_f32<T>(buf[d]);
      }
    }
    __syncthreads();  // buf is reused in the next round
  }
}

#define DEFINE_ROPE(SUF, T)                                                                        \
  extern "C" int jv_qk_norm_rope_write_##SUF(                                                      \
      void* qkv, const int* positions, const int* slot_mapping, const float* q_w,                  \
      const float* k_w, float eps, const float* inv_freq, int rotary_dim, int interleaved,         \
      void* k_pages, void* v_pages, int page_size, int n_tokens, int nq, int nkv, int D,           \
      void* stream) {                                                                              \
    if (n_tokens <= 0) return 0;                                                                   \
    if (D > ROPE_MAX_D || rotary_dim > D || (rotary_dim & 1)) return (int)hipErrorInvalidValue;    \
    const int waves = 4;                                                                           \
    hipLaunchKernelGGL(qk_norm_rope_write_kernel<T>, dim3(n_tokens), dim3(waves * JV_WAVE),        \
                       waves * D * sizeof(float), (hipStream_t)stream, (T*)qkv, positions,         \
                       slot_mapping, q_w, k_w, eps, inv_freq, rotary_dim, interleaved,             \
                       (T*)k_pages, (T*)v_pages, page_size, nq, nkv, D);                           \
    return JV_LAUNCH_CHECK();                                                                      \
  }

DEFINE_ROPE(bf16, bf16_t)
DEFINE_ROPE(f32, float)
