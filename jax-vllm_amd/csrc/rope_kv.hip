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
    int nkv, int D, int v_elsewhere) {
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
  if (is_v && store && !v_elsewhere) {  // v head: copied to its (transposed) page
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
// No load sits inside a branch (one that does makes the compiler wait, where the branch ends, for
// every load in flight, and a step of few tokens is a chain of memory round trips): what is not
// there (no rotation, no norm weight, no slot) is read from the row itself and given no weight.
template <typename T, int E, int NP>
__global__ void __launch_bounds__(256) qk_norm_rope_write_fast_kernel(
    T* __restrict__ qkv, const float* __restrict__ parts, long long part_stride,
    const int* __restrict__ slot_mapping, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin, int rotary_dim,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size, int nq, int nkv,
    int heads_per_wave, int walk_heads) {
  constexpr int D = E * 64;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const long long t = blockIdx.x;
  const int n_heads = nq + 2 * nkv;
  T* row = qkv + t * (long long)n_heads * D;
  const int half = rotary_dim / 2, HE = half / 64;   // pair (e, e + HE) for e < HE
  const int h0 = (blockIdx.y * 4 + wid) * heads_per_wave;
  if (h0 >= walk_heads) return;                       // the whole wave
  // everything that does not depend on the head: slot, cos/sin of this lane's pair indices
  // the slot through the vector unit (an index the compiler cannot see through): a scalar load would be
  // waited for before the loads below are even asked for
  int lane_zero;
  asm volatile("v_mov_b32 %0, 0" : "=v"(lane_zero));
  const int* slot_at = slot_mapping ? slot_mapping + t : (const int*)row;
  const int slot_raw = slot_at[lane_zero];
  float cs[E], sn[E];
  {
    // without a table: the row itself, read as floats (at least 3 heads of D elements of 2 bytes: long enough)
    const float* cp = cos_sin ? cos_sin + t * rotary_dim + lane : (const float*)row + lane;
    const int hh = cos_sin ? half : 0;
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int ee = e < HE ? e : 0;
      cs[e] = cp[ee * 64];
      sn[e] = cp[hh + ee * 64];
    }
  }
  for (int head = h0; head < h0 + heads_per_wave && head < walk_heads; ++head) {
    T* x = row + (long long)head * D;
    float v[E], wv[E];
    {  // the norm weights are asked for together with the head, not after its reduction
      const float* w0 = head < nq ? q_w : (head < nq + nkv ? k_w : nullptr);
      const float* wp = (w0 ? w0 : (const float*)row) + lane;
#pragma unroll
      for (int e = 0; e < E; ++e) wv[e] = wp[e * 64];      // used only where there is a weight
    }
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
    // the slot is looked at only here, after every load of the head has been asked for
    const long long slot = slot_mapping ? (long long)__builtin_amdgcn_readfirstlane(slot_raw) : -1;
    const bool store = (slot >= 0) && (k_pages != nullptr);
    const long long page = store ? slot / page_size : 0;
    const int off = store ? (int)(slot - page * page_size) : 0;
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

// The v heads of many tokens into their transposed pages [page][kv head][D][slot].  Token by token
// every element would be a store of its own, 2 bytes every `page_size` elements; here a block takes
// 16 consecutive tokens of one kv head through LDS and writes, for every element of the head, 8
// tokens at once (16 bytes) wherever 8 consecutive tokens have 8 consecutive slots that start at a
// multiple of 8 (the usual case for a prompt), and element by element elsewhere.
template <typename T> struct alignas(16) Pack8 { T v[8]; };

template <typename T>
__global__ void __launch_bounds__(256) v_pages_write_kernel(
    const T* __restrict__ qkv, const int* __restrict__ slot_mapping, T* __restrict__ v_pages, int page_size,
    int n_tokens, int nq, int nkv, int D) {
  constexpr int EP = 16 / (int)sizeof(T);          // elements of a 16-byte piece
  extern __shared__ __attribute__((aligned(16))) unsigned char v_tile_mem[];
  T* tile = (T*)v_tile_mem;                        // [16][D + EP]
  const int LROW = D + EP;
  const int t0 = blockIdx.x * 16, kvh = blockIdx.y;
  const long long row_stride = (long long)(nq + 2 * nkv) * D;
  const T* src = qkv + (long long)(nq + nkv + kvh) * D;
  const int ppt = D / EP;
  for (int p = threadIdx.x; p < 16 * ppt; p += 256) {
    const int j = p / ppt, c = (p - j * ppt) * EP;
    if (t0 + j < n_tokens) *(uint4*)(tile + j * LROW + c) = *(const uint4*)(src + (t0 + j) * row_stride + c);
  }
  __syncthreads();
  for (int item = threadIdx.x; item < 2 * D; item += 256) {
    const int half = item / D, d = item - half * D;
    const int tb = t0 + half * 8;
    if (tb >= n_tokens) continue;
    const int s0 = slot_mapping[tb];
    bool run = s0 >= 0 && (s0 & 7) == 0 && tb + 8 <= n_tokens;
    if (run) {
#pragma unroll
      for (int j = 1; j < 8; ++j) run = run && slot_mapping[tb + j] == s0 + j;
    }
    const T* col = tile + (half * 8) * LROW + d;
    if (run) {
      const long long page = s0 / page_size;
      const int off = (int)(s0 - page * page_size);
      Pack8<T> v;
#pragma unroll
      for (int j = 0; j < 8; ++j) v.v[j] = col[j * LROW];
      *(Pack8<T>*)(v_pages + ((page * nkv + kvh) * D + d) * (long long)page_size + off) = v;
    } else {
      for (int j = 0; j < 8 && tb + j < n_tokens; ++j) {
        const int s = slot_mapping[tb + j];
        if (s < 0) continue;
        const long long page = s / page_size;
        const int off = (int)(s - page * page_size);
        v_pages[((page * nkv + kvh) * D + d) * (long long)page_size + off] = col[j * LROW];
      }
    }
  }
}

// Full rotation (or none) with half-split pairing, head size 64, 128 or 256, any number of tokens:
// a lane holds two 16-byte pieces of a head, the same places of its two halves, so both numbers
// of every rotation pair sit in one lane and a head takes only D/16 lanes (bf16): a wave prepares
// 64 / (D/16) heads of one token with two 16-byte loads and stores a lane.  q in place, k to its
// page; the v heads are written by v_pages_write_kernel.
template <typename T, int D>
__global__ void __launch_bounds__(256) qk_norm_rope_write_wide_kernel(
    T* __restrict__ qkv, const int* __restrict__ slot_mapping, const float* __restrict__ q_w,
    const float* __restrict__ k_w, float eps, const float* __restrict__ cos_sin, T* __restrict__ k_pages,
    int page_size, int n_tokens, int nq, int nkv) {
  constexpr int EP = 16 / (int)sizeof(T), HALF = D / 2, LPH = HALF / EP, HPW = 64 / LPH;
  static_assert(LPH >= 1 && LPH <= 64 && (LPH & (LPH - 1)) == 0, "lanes per head must be a power of two");
  const int lane = threadIdx.x & 63;
  const int walk = nq + nkv, groups = (walk + HPW - 1) / HPW;
  const long long item = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (item >= (long long)n_tokens * groups) return;
  const long long t = item / groups;
  const int grp = (int)(item - t * groups);
  const int head = grp * HPW + lane / LPH, p = (lane % LPH) * EP;
  const bool is_q = head < nq;
  const long long slot = slot_mapping ? (long long)slot_mapping[t] : -1;
  const bool store = (slot >= 0) && (k_pages != nullptr);
  const bool work = head < walk && (is_q || store);   // a k head that nobody will read is skipped
  const long long page = store ? slot / page_size : 0;
  const int off = store ? (int)(slot - page * page_size) : 0;
  T* x = qkv + (t * (nq + 2 * nkv) + (head < walk ? head : 0)) * (long long)D + p;
  // everything is asked for before anything is looked at
  struct alignas(16) Piece { T v[EP]; };
  const Piece pa = *(const Piece*)x, pb = *(const Piece*)(x + HALF);
  const float* w = is_q ? q_w : k_w;
  float wa[EP], wb[EP], cs[EP], sn[EP];
  auto load_floats = [&](const float* src, float (&dst)[EP], float otherwise) {   // 16-byte loads; src is aligned
#pragma unroll
    for (int e = 0; e < EP; e += 4) {
      const float4 v = src ? *(const float4*)(src + e) : make_float4(otherwise, otherwise, otherwise, otherwise);
      dst[e] = v.x; dst[e + 1] = v.y; dst[e + 2] = v.z; dst[e + 3] = v.w;
    }
  };
  load_floats(w ? w + p : nullptr, wa, 1.f);
  load_floats(w ? w + HALF + p : nullptr, wb, 1.f);
  load_floats(cos_sin ? cos_sin + t * D + p : nullptr, cs, 1.f);
  load_floats(cos_sin ? cos_sin + t * D + HALF + p : nullptr, sn, 0.f);
  float a[EP], b[EP], ss = 0.f;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    a[e] = to_f32(pa.v[e]);
    b[e] = to_f32(pb.v[e]);
    ss += a[e] * a[e] + b[e] * b[e];
  }
#pragma unroll
  for (int o = LPH / 2; o > 0; o >>= 1) ss += __shfl_xor(ss, o, JV_WAVE);
  if (!work) return;
  if (w) {
    const float inv = rsqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < EP; ++e) {
      a[e] = a[e] * inv * wa[e];
      b[e] = b[e] * inv * wb[e];
    }
  }
  Piece oa, ob;
#pragma unroll
  for (int e = 0; e < EP; ++e) {
    oa.v[e] = from_f32<T>(a[e] * cs[e] - b[e] * sn[e]);
    ob.v[e] = from_f32<T>(b[e] * cs[e] + a[e] * sn[e]);
  }
  T* dst = is_q ? x : k_pages + ((page * nkv + (head - nq)) * page_size + off) * (long long)D + p;
  *(Piece*)dst = oa;
  *(Piece*)(dst + HALF) = ob;
}

template <typename T, int D>
static int launch_rope_wide(void* qkv, const int* slot_mapping, const float* q_w, const float* k_w, float eps,
                            const float* cos_sin, void* k_pages, int page_size, int n_tokens, int nq, int nkv,
                            void* stream) {
  constexpr int HPW = 64 / (D / 2 / (16 / (int)sizeof(T)));
  const long long items = (long long)n_tokens * ((nq + nkv + HPW - 1) / HPW);
  if ((items + 3) / 4 > 0x7fffffffll) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL((qk_norm_rope_write_wide_kernel<T, D>), dim3((unsigned)((items + 3) / 4)), dim3(256), 0,
                     (hipStream_t)stream, (T*)qkv, slot_mapping, q_w, k_w, eps, cos_sin, (T*)k_pages, page_size,
                     n_tokens, nq, nkv);
  return JV_LAUNCH_CHECK();
}

// Whether the v heads of a step go through v_pages_write_kernel: many tokens, and sizes that keep
// its 16-byte pieces aligned.
template <typename T>
static bool v_written_by_tile(const void* k_pages, int n_tokens, int page_size, int D) {
  return k_pages != nullptr && n_tokens >= 256 && page_size % 8 == 0 && D % (16 / (int)sizeof(T)) == 0;
}

template <typename T>
static int launch_v_pages_write(const void* qkv, const int* slot_mapping, void* v_pages, int page_size,
                                int n_tokens, int nq, int nkv, int D, void* stream) {
  if (nkv > 65535) return (int)hipErrorInvalidValue;
  const size_t shmem = (size_t)16 * (D + 16 / sizeof(T)) * sizeof(T);
  hipLaunchKernelGGL(v_pages_write_kernel<T>, dim3((n_tokens + 15) / 16, nkv), dim3(256), shmem,
                     (hipStream_t)stream, (const T*)qkv, slot_mapping, (T*)v_pages, page_size, n_tokens, nq, nkv, D);
  return JV_LAUNCH_CHECK();
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
    const bool v_tile = v_written_by_tile<T>(k_pages, n_tokens, page_size, D);                     \
    if (v_tile) {                                                                                  \
      const int e = launch_v_pages_write<T>(qkv, slot_mapping, v_pages, page_size, n_tokens, nq,   \
                                            nkv, D, stream);                                       \
      if (e) return e;                                                                             \
    }                                                                                              \
    const int walk = v_tile ? nq + nkv : n_heads;                                                  \
    if (v_tile && !interleaved && (!cos_sin || rotary_dim == D) && (D == 64 || D == 128 || D == 256)) {  \
      if (D == 64) return launch_rope_wide<T, 64>(qkv, slot_mapping, q_w, k_w, eps, cos_sin, k_pages,    \
                                                  page_size, n_tokens, nq, nkv, stream);           \
      if (D == 128) return launch_rope_wide<T, 128>(qkv, slot_mapping, q_w, k_w, eps, cos_sin, k_pages,  \
                                                    page_size, n_tokens, nq, nkv, stream);         \
      return launch_rope_wide<T, 256>(qkv, slot_mapping, q_w, k_w, eps, cos_sin, k_pages, page_size, \
                                      n_tokens, nq, nkv, stream);                                  \
    }                                                                                              \
    if ((D == 128 || D == 256) && !interleaved && (!cos_sin || (half % 64 == 0 && half > 0))) {    \
      /* many tokens: a wave walks several heads; few tokens: one head per wave for parallelism */ \
      const int hpw = n_tokens >= 256 ? (walk + 3) / 4 : 1;                                        \
      const int gy = (walk + 4 * hpw - 1) / (4 * hpw);                                             \
      if (D == 128)                                                                                \
        hipLaunchKernelGGL((qk_norm_rope_write_fast_kernel<T, 2, 0>), dim3(n_tokens, gy),          \
                           dim3(256), 0, (hipStream_t)stream, (T*)qkv, (const float*)nullptr, 0ll, \
                           slot_mapping, q_w, k_w, eps, cos_sin, rotary_dim, (T*)k_pages,          \
                           (T*)v_pages, page_size, nq, nkv, hpw, walk);                            \
      else                                                                                         \
        hipLaunchKernelGGL((qk_norm_rope_write_fast_kernel<T, 4, 0>), dim3(n_tokens, gy),          \
                           dim3(256), 0, (hipStream_t)stream, (T*)qkv, (const float*)nullptr, 0ll, \
                           slot_mapping, q_w, k_w, eps, cos_sin, rotary_dim, (T*)k_pages,          \
                           (T*)v_pages, page_size, nq, nkv, hpw, walk);                            \
      return JV_LAUNCH_CHECK();                                                                    \
    }                                                                                              \
    hipLaunchKernelGGL(qk_norm_rope_write_kernel<T>, dim3(n_tokens, (walk + 3) / 4), dim3(256),    \
                       4 * D * sizeof(float), (hipStream_t)stream, (T*)qkv, slot_mapping, q_w,     \
                       k_w, eps, cos_sin, rotary_dim, interleaved, (T*)k_pages, (T*)v_pages,       \
                       page_size, nq, nkv, D, v_tile ? 1 : 0);                                     \
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
                     rotary_dim, (T*)k_pages, (T*)v_pages, page_size, nq, nkv, hpw, n_heads);
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
