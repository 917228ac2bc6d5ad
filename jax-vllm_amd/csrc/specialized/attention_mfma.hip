// Paged causal attention on the matrix cores (bf16 in, float accumulate, float softmax),
// specialised at compile time for one head size: -DJV_HEAD_DIM=<multiple of 16, <= 256>.
//
// Cache layout:  K pages [page][kv_head][slot][D]      (a key's D elements contiguous)
//                V pages [page][kv_head][D][slot]      (transposed: a page's keys contiguous per d)
// page_size must be a multiple of 8, so that 8 consecutive keys starting at a multiple of 8
// lie in one page and the V layout gives 16 aligned bytes.
//
// Both kernels compute the transposed products so that every lane's numbers belong to one
// query row (row statistics are per-lane scalars):
//   S^T[key][row] = K * Q^T        v_mfma_f32_16x16x32_bf16, A = K rows, B = Q rows
//   O^T[d][row]  += V^T * P^T      A = V^T (8 keys per lane at one d), B = P^T taken straight
//                                  from the S^T accumulators (no shuffle, no LDS round trip)
// In the 16x16x32 layout lane l holds, for A and B alike, row/column l%16 and the 8
// contraction indices (l/16)*8..+8; the accumulator holds rows (l/16)*4..+4 of column l%16.
// The contraction index may be permuted freely if A and B agree, which is what lets two
// 16-key accumulators (4 keys each per lane) feed one 32-key P^T operand.
//
// Rows of a work item are the (query, head-in-group) pairs of one request and one kv head:
// row m = query_index * G + head_in_group, G = q heads per kv head; any G works.
//   prefill kernel: 64 rows per block (4 waves x 16), K/V tiles of 64 keys staged in LDS and
//                   shared by the 4 waves; causal limit and window per row.
//   decode kernel:  one query per request; each of the 4 waves streams its own 32-key tiles
//                   straight from global memory into MFMA operands (no LDS), the waves'
//                   partial (max, sum, acc) are merged in LDS; with num_splits > 1 several
//                   blocks share a request's keys and a second kernel merges their partials.
#include "../common.h"

#ifndef JV_HEAD_DIM
#error "compile with -DJV_HEAD_DIM=<head size>"
#endif
static_assert(JV_HEAD_DIM % 16 == 0 && JV_HEAD_DIM >= 16 && JV_HEAD_DIM <= 256, "head size");

constexpr int D = JV_HEAD_DIM;
constexpr int NDT = D / 16;                // 16-wide tiles of the head dimension (output)
constexpr int DK = (D + 31) / 32 * 32;     // head dimension padded to the QK contraction step
constexpr int NKS = DK / 32;
constexpr int BN = 64;                     // keys per LDS tile (prefill)
constexpr int KS_STRIDE = DK + 8;          // bf16 elements per key row in LDS
constexpr int VT_STRIDE = BN + 16;         // bf16 elements per d row in LDS

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

struct AttnArgs {
  bf16_t* out;                // [tokens, nq * D]
  const bf16_t* q;            // row t at q + t * q_row_stride, head h at + h * D
  long long q_row_stride;
  const bf16_t* k_pages;
  const bf16_t* v_pages;
  const int* block_tables;    // [requests, table_stride]
  int table_stride;
  const int* cu_seqlens;      // [requests + 1]
  const int* context_lens;    // [requests] keys stored before this step
  const int* work;            // prefill: [n_work][2] = (request, first row); decode: [n_work] = request
  int page_size, nq, nkv;
  float scale_log2;           // softmax scale * log2(e)
  int window;                 // <= 0: none
  // decode only
  int num_splits;
  float* part_acc;            // [n_work, nq, num_splits, D]
  float* part_ml;             // [n_work, nq, num_splits, 2] (max, sum)
};

// ------------------------------------------------------------------------------------ prefill
__global__ void __launch_bounds__(256) attn_prefill_kernel(AttnArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BN * KS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D * VT_STRIDE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lc = lane >> 4;
  const int r = p.work[2 * blockIdx.x], m0 = p.work[2 * blockIdx.x + 1];
  const int g = blockIdx.y;
  const int G = p.nq / p.nkv, P = p.page_size;
  const int q_start = p.cu_seqlens[r], q_len = p.cu_seqlens[r + 1] - q_start;
  const int ctx = p.context_lens[r];
  const int M = q_len * G;
  const int* table = p.block_tables + (long long)r * p.table_stride;

  const int row = m0 + wave * 16 + li;
  const bool row_ok = row < M;
  const int qi = row_ok ? row / G : 0, hg = row_ok ? row - (row / G) * G : 0;
  const int pos = ctx + qi;

  bf16x8 qf[NKS];
  {
    const bf16_t* qrow = p.q + (long long)(q_start + qi) * p.q_row_stride + (long long)(g * G + hg) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int d0 = ks * 32 + lc * 8;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row_ok && d0 < D) v = *(const bf16x8*)(qrow + d0);
      qf[ks] = v;
    }
  }
  // key range of the block and of this wave
  const int last_row = (M < m0 + 64 ? M : m0 + 64) - 1;
  const int kv_end = ctx + last_row / G + 1;
  int kv_begin = 0;
  if (p.window > 0) {
    kv_begin = ctx + m0 / G - p.window + 1;
    if (kv_begin < 0) kv_begin = 0;
  }
  const int wave_first = m0 + wave * 16;
  const int wave_last = (M < wave_first + 16 ? M : wave_first + 16) - 1;
  const int wave_kv_end = wave_first < M ? ctx + wave_last / G + 1 : 0;
  int wave_kv_begin = 0;
  if (p.window > 0 && wave_first < M) {
    wave_kv_begin = ctx + wave_first / G - p.window + 1;
    if (wave_kv_begin < 0) wave_kv_begin = 0;
  }

  float m_run = -INFINITY, l_lane = 0.f;
  f32x4 acc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int j0 = kv_begin / BN * BN; j0 < kv_end; j0 += BN) {
    // ---- stage K [64 keys][DK] and V^T [D][64 keys]; keys at or past kv_end become zeros
    for (int c = tid; c < BN * (DK / 8); c += 256) {
      const int key = c / (DK / 8), dc = c - key * (DK / 8);
      const int j = j0 + key;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (j < kv_end && dc * 8 < D) {
        const long long page = table[j / P];
        v = *(const bf16x8*)(p.k_pages + ((page * p.nkv + g) * P + (j % P)) * (long long)D + dc * 8);
      }
      *(bf16x8*)(Ks + key * KS_STRIDE + dc * 8) = v;
    }
    for (int c = tid; c < D * (BN / 8); c += 256) {
      const int d = c / (BN / 8), kc = c - d * (BN / 8);
      const int j = j0 + kc * 8;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (j < kv_end) {
        const long long page = table[j / P];
        v = *(const bf16x8*)(p.v_pages + ((page * p.nkv + g) * D + d) * (long long)P + (j % P));
        if (j + 8 > kv_end) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (j + e >= kv_end) v[e] = (bf16_t)0.f;
        }
      }
      *(bf16x8*)(Vt + d * VT_STRIDE + kc * 8) = v;
    }
    __syncthreads();

    if (j0 < wave_kv_end && j0 + BN > wave_kv_begin) {
      f32x4 s[4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const bf16x8 a = *(const bf16x8*)(Ks + (kt * 16 + li) * KS_STRIDE + ks * 32 + lc * 8);
          s[kt] = mfma16(a, qf[ks], s[kt]);
        }
      }
      float tmax = -INFINITY;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int j = j0 + kt * 16 + lc * 4 + e;
          const bool ok = row_ok && j <= pos && (p.window <= 0 || j > pos - p.window);
          const float v = ok ? s[kt][e] * p.scale_log2 : -INFINITY;
          s[kt][e] = v;
          tmax = fmaxf(tmax, v);
        }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);
      const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
      const float alpha = fast_exp2(m_run - m_use);
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float pv = fast_exp2(s[kt][e] - m_use);
          s[kt][e] = pv;
          psum += pv;
        }
      l_lane = l_lane * alpha + psum;
      m_run = m_new;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) acc[dt] *= alpha;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        bf16x8 b;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          b[e] = (bf16_t)s[2 * kk][e];
          b[4 + e] = (bf16_t)s[2 * kk + 1][e];
        }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
          const bf16_t* vrow = Vt + (dt * 16 + li) * VT_STRIDE + lc * 4;
          const bf16x4 a0 = *(const bf16x4*)(vrow + (2 * kk) * 16);
          const bf16x4 a1 = *(const bf16x4*)(vrow + (2 * kk + 1) * 16);
          const bf16x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
          acc[dt] = mfma16(a, b, acc[dt]);
        }
      }
    }
    __syncthreads();
  }

  float l = l_lane + __shfl_xor(l_lane, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (row_ok) {
    const float inv = 1.f / l;
    bf16_t* o = p.out + (long long)(q_start + qi) * p.nq * D + (long long)(g * G + hg) * D + lc * 4;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16_t)(acc[dt][e] * inv);
      *(bf16x4*)(o + dt * 16) = v;
    }
  }
}

// ------------------------------------------------------------------------------------ decode
constexpr int BND = 32;  // keys per wave iteration

__global__ void __launch_bounds__(256) attn_decode_kernel(AttnArgs p) {
  extern __shared__ float smem[];  // per wave: m[16], l[16], acc[16][D]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lc = lane >> 4;
  const int G = p.nq / p.nkv, P = p.page_size;
  const int mt_per_head = (G + 15) / 16;
  const int w = blockIdx.x;
  const int r = p.work[w];
  const int g = blockIdx.y / mt_per_head, mt = blockIdx.y - g * mt_per_head;
  const int split = blockIdx.z;
  const int tok = p.cu_seqlens[r];
  const int pos = p.context_lens[r];      // the query's position; keys 0..pos are stored
  const int kv_len = pos + 1;
  int kv_begin = 0;
  if (p.window > 0 && pos - p.window + 1 > 0) kv_begin = pos - p.window + 1;
  const int* table = p.block_tables + (long long)r * p.table_stride;

  const int hg = mt * 16 + li;
  const bool row_ok = hg < G;
  bf16x8 qf[NKS];
  {
    const bf16_t* qrow = p.q + (long long)tok * p.q_row_stride + (long long)(g * G + (row_ok ? hg : 0)) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int d0 = ks * 32 + lc * 8;
      bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
      if (row_ok && d0 < D) v = *(const bf16x8*)(qrow + d0);
      qf[ks] = v;
    }
  }
  // tiles of this split, shared out to the 4 waves round-robin
  const int t_first = kv_begin / BND, t_total = (kv_len + BND - 1) / BND - t_first;
  const int per_split = (t_total + p.num_splits - 1) / p.num_splits;
  const int t_lo = t_first + split * per_split;
  int t_hi = t_lo + per_split;
  if (t_hi > t_first + t_total) t_hi = t_first + t_total;

  float m_run = -INFINITY, l_lane = 0.f;
  f32x4 acc[NDT];
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  for (int t = t_lo + wave; t < t_hi; t += 4) {
    const int j0 = t * BND;
    // K operand: lane (key li of sub-tile kt, chunk lc) <- 8 consecutive d of that key
    bf16x8 kf[2][NKS];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int j = j0 + kt * 16 + li;
      const bool ok = j < kv_len;
      const long long page = ok ? table[j / P] : 0;
      const bf16_t* krow = p.k_pages + ((page * p.nkv + g) * P + (ok ? j % P : 0)) * (long long)D;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = ks * 32 + lc * 8;
        bf16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (ok && d0 < D) v = *(const bf16x8*)(krow + d0);
        kf[kt][ks] = v;
      }
    }
    // V^T operand: lane (d = dt*16 + li, chunk lc) <- keys kt*16 + lc*4 .. +4 of that d
    bf16x4 vf[2][NDT];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int j = j0 + kt * 16 + lc * 4;
      const bool ok = j < kv_len;
      const long long page = ok ? table[j / P] : 0;
      const bf16_t* vbase = p.v_pages + (page * p.nkv + g) * (long long)D * P + (ok ? j % P : 0);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        bf16x4 v = {0, 0, 0, 0};
        if (ok) {
          v = *(const bf16x4*)(vbase + (long long)(dt * 16 + li) * P);
          if (j + 4 > kv_len) {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (j + e >= kv_len) v[e] = (bf16_t)0.f;
          }
        }
        vf[kt][dt] = v;
      }
    }
    f32x4 s[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      s[kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) s[kt] = mfma16(kf[kt][ks], qf[ks], s[kt]);
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int j = j0 + kt * 16 + lc * 4 + e;
        const bool ok = row_ok && j <= pos && j >= kv_begin;
        const float v = ok ? s[kt][e] * p.scale_log2 : -INFINITY;
        s[kt][e] = v;
        tmax = fmaxf(tmax, v);
      }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    const float alpha = fast_exp2(m_run - m_use);
    float psum = 0.f;
    bf16x8 b;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float pv = fast_exp2(s[kt][e] - m_use);
        psum += pv;
        b[kt * 4 + e] = (bf16_t)pv;
      }
    l_lane = l_lane * alpha + psum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      const bf16x4 a0 = vf[0][dt], a1 = vf[1][dt];
      const bf16x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      acc[dt] = mfma16(a, b, acc[dt] * alpha);
    }
  }

  // ---- merge the 4 waves through LDS
  float l = l_lane + __shfl_xor(l_lane, 16, 64);
  l += __shfl_xor(l, 32, 64);
  float* sm = smem + wave * (32 + 16 * D);
  if (lc == 0) {
    sm[li] = m_run;
    sm[16 + li] = l;
  }
#pragma unroll
  for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
    for (int e = 0; e < 4; ++e) sm[32 + li * D + dt * 16 + lc * 4 + e] = acc[dt][e];
  __syncthreads();
  const int rows = G - mt * 16 < 16 ? G - mt * 16 : 16;
  for (int idx = tid; idx < rows * D; idx += 256) {
    const int rr = idx / D, d = idx - rr * D;
    float mx = -INFINITY;
#pragma unroll
    for (int ww = 0; ww < 4; ++ww) mx = fmaxf(mx, smem[ww * (32 + 16 * D) + rr]);
    float num = 0.f, den = 0.f;
    if (mx != -INFINITY) {
#pragma unroll
      for (int ww = 0; ww < 4; ++ww) {
        const float* s2 = smem + ww * (32 + 16 * D);
        const float f = fast_exp2(s2[rr] - mx);
        num += s2[32 + rr * D + d] * f;
        den += s2[16 + rr] * f;
      }
    }
    const int head = g * G + mt * 16 + rr;
    if (p.num_splits == 1) {
      p.out[(long long)tok * p.nq * D + (long long)head * D + d] = (bf16_t)(num / den);
    } else {
      const long long slot = ((long long)w * p.nq + head) * p.num_splits + split;
      p.part_acc[slot * D + d] = num;
      if (d == 0) {
        p.part_ml[slot * 2] = mx;
        p.part_ml[slot * 2 + 1] = den;
      }
    }
  }
}

// merges the splits of one (request, head): grid (n_work, nq), D threads (rounded up to 64)
__global__ void attn_decode_merge_kernel(AttnArgs p) {
  const int w = blockIdx.x, head = blockIdx.y, d = threadIdx.x;
  const int r = p.work[w];
  const int tok = p.cu_seqlens[r];
  const long long base = ((long long)w * p.nq + head) * p.num_splits;
  float mx = -INFINITY;
  for (int s = 0; s < p.num_splits; ++s) mx = fmaxf(mx, p.part_ml[(base + s) * 2]);
  if (d >= D) return;
  float num = 0.f, den = 0.f;
  for (int s = 0; s < p.num_splits; ++s) {
    const float ms = p.part_ml[(base + s) * 2];
    if (ms == -INFINITY) continue;
    const float f = fast_exp2(ms - mx);
    num += p.part_acc[(base + s) * D + d] * f;
    den += p.part_ml[(base + s) * 2 + 1] * f;
  }
  p.out[(long long)tok * p.nq * D + (long long)head * D + d] = (bf16_t)(num / den);
}

// ------------------------------------------------------------------------------------ entry points
static int check_common(const AttnArgs& a) {
  if (a.page_size <= 0 || a.page_size % 8 != 0) return (int)hipErrorInvalidValue;
  if (a.nkv <= 0 || a.nq % a.nkv != 0) return (int)hipErrorInvalidValue;
  return 0;
}

extern "C" int jv_attn_head_dim() { return D; }

extern "C" int jv_attn_prefill(void* out, const void* q, long long q_row_stride, const void* k_pages,
                               const void* v_pages, const int* block_tables, int table_stride,
                               const int* cu_seqlens, const int* context_lens, const int* work,
                               int n_work, int page_size, int nq, int nkv, float scale, int window,
                               void* stream) {
  if (n_work <= 0) return 0;
  AttnArgs a{};
  a.out = (bf16_t*)out; a.q = (const bf16_t*)q; a.q_row_stride = q_row_stride;
  a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
  a.block_tables = block_tables; a.table_stride = table_stride;
  a.cu_seqlens = cu_seqlens; a.context_lens = context_lens; a.work = work;
  a.page_size = page_size; a.nq = nq; a.nkv = nkv;
  a.scale_log2 = scale * 1.4426950408889634f; a.window = window; a.num_splits = 1;
  if (int e = check_common(a)) return e;
  if (nkv > 65535) return (int)hipErrorInvalidValue;
  hipLaunchKernelGGL(attn_prefill_kernel, dim3(n_work, nkv), dim3(256), 0, (hipStream_t)stream, a);
  return JV_LAUNCH_CHECK();
}

// floats of scratch the decode entry point needs for (n_work, nq, num_splits)
extern "C" long long jv_attn_decode_scratch_floats(int n_work, int nq, int num_splits) {
  return num_splits > 1 ? (long long)n_work * nq * num_splits * (D + 2) : 0;
}

extern "C" int jv_attn_decode(void* out, const void* q, long long q_row_stride, const void* k_pages,
                              const void* v_pages, const int* block_tables, int table_stride,
                              const int* cu_seqlens, const int* context_lens, const int* work,
                              int n_work, int page_size, int nq, int nkv, float scale, int window,
                              int num_splits, float* scratch, void* stream) {
  if (n_work <= 0) return 0;
  AttnArgs a{};
  a.out = (bf16_t*)out; a.q = (const bf16_t*)q; a.q_row_stride = q_row_stride;
  a.k_pages = (const bf16_t*)k_pages; a.v_pages = (const bf16_t*)v_pages;
  a.block_tables = block_tables; a.table_stride = table_stride;
  a.cu_seqlens = cu_seqlens; a.context_lens = context_lens; a.work = work;
  a.page_size = page_size; a.nq = nq; a.nkv = nkv;
  a.scale_log2 = scale * 1.4426950408889634f; a.window = window;
  a.num_splits = num_splits < 1 ? 1 : num_splits;
  if (int e = check_common(a)) return e;
  if (a.num_splits > 1) {
    if (!scratch) return (int)hipErrorInvalidValue;
    a.part_acc = scratch;
    a.part_ml = scratch + (long long)n_work * nq * a.num_splits * D;
  }
  const int G = nq / nkv, mt_per_head = (G + 15) / 16;
  if ((long long)nkv * mt_per_head > 65535 || a.num_splits > 65535) return (int)hipErrorInvalidValue;
  const size_t shmem = 4 * (32 + 16 * D) * sizeof(float);
  if (shmem > 64 * 1024) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_decode_kernel,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)shmem);
    if (e != hipSuccess) return (int)e;
  }
  hipLaunchKernelGGL(attn_decode_kernel, dim3(n_work, nkv * mt_per_head, a.num_splits), dim3(256),
                     shmem, (hipStream_t)stream, a);
  int e = JV_LAUNCH_CHECK();
  if (e) return e;
  if (a.num_splits > 1) {
    hipLaunchKernelGGL(attn_decode_merge_kernel, dim3(n_work, nq), dim3((D + 63) / 64 * 64), 0,
                       (hipStream_t)stream, a);
    e = JV_LAUNCH_CHECK();
  }
  return e;
}
