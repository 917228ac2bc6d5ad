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
//   prefill kernel: 128 rows per block (4 waves x 2 row tiles of 16; 64 rows for heads above 128), K/V tiles of 64 keys staged
//                   in LDS and shared by the 4 waves; causal limit and window per row.
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
constexpr int VT_STRIDE = BN + 8;          // bf16 elements per d row in LDS (rows 16-byte aligned, 4 banks apart)

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f32x4 mfma16(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}
__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// j -> (page index in the table, slot in the page); a shift and a mask when the page size is a
// power of two (page_shift >= 0), a division otherwise.
struct PageSplit {
  int P, shift;
  __device__ __forceinline__ int index(int j) const { return shift >= 0 ? (j >> shift) : j / P; }
  __device__ __forceinline__ int slot(int j) const { return shift >= 0 ? (j & (P - 1)) : j % P; }
};

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
  const int* work;            // prefill: [n_work][2] = (request, first row of a block of 128); decode: [n_work] = request
  int page_size, page_shift, nq, nkv;   // page_shift: log2(page_size) or -1
  float scale_log2;           // softmax scale * log2(e)
  int window;                 // <= 0: none
  // decode only
  int num_splits;
  float* part_acc;            // [n_work, nq, num_splits, D]
  float* part_ml;             // [n_work, nq, num_splits, 2] (max, sum)
};

// ------------------------------------------------------------------------------------ prefill
// 128 rows per block: 4 waves x 2 row tiles of 16 (one row tile, 64 rows, for head sizes above
// 128).  Every K fragment and every V^T fragment read
// from LDS feeds both row tiles of the wave.  The next tile's K/V are fetched from global memory
// into registers while the current tile is multiplied, and written to LDS between two barriers.
// Keys are masked only on tiles that cross a row's causal limit or window edge.
constexpr int RT = D <= 128 ? 2 : 1;        // row tiles per wave (one for large heads: registers)
constexpr int BM = 4 * RT * 16;            // rows per block
constexpr int KCH = BN * (DK / 8);         // 16-byte pieces of a K tile
constexpr int VCH = D * (BN / 8);          // 16-byte pieces of a V^T tile
constexpr int KPT = (KCH + 255) / 256;     // pieces per thread
constexpr int VPT = (VCH + 255) / 256;
constexpr int TBL_MAX = 2048;              // page-table entries a block keeps in LDS

#if JV_HEAD_DIM <= 128
#define PREFILL_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2, 2)))  // two waves per SIMD: one's softmax hides the other's MFMA
#else
#define PREFILL_OCCUPANCY
#endif
__global__ void __launch_bounds__(256) PREFILL_OCCUPANCY attn_prefill_kernel(AttnArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BN * KS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D * VT_STRIDE];
  __shared__ int page_ids[TBL_MAX];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lc = lane >> 4;
  const int r = p.work[2 * blockIdx.x], m0 = p.work[2 * blockIdx.x + 1];
  const int g = blockIdx.y;
  const int G = p.nq / p.nkv, P = p.page_size;
  const PageSplit ps{P, p.page_shift};
  const int q_start = p.cu_seqlens[r], q_len = p.cu_seqlens[r + 1] - q_start;
  const int ctx = p.context_lens[r];
  const int M = q_len * G;
  const int* gtable = p.block_tables + (long long)r * p.table_stride;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // this lane's rows: one per row tile
  int row[RT], qi[RT], hg[RT], pos[RT];
  bool row_ok[RT];
  bf16x8 qf[RT][NKS];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    row[t] = m0 + (wave * RT + t) * 16 + li;
    row_ok[t] = row[t] < M;
    qi[t] = row_ok[t] ? row[t] / G : 0;
    hg[t] = row_ok[t] ? row[t] - qi[t] * G : 0;
    pos[t] = ctx + qi[t];
    const bf16_t* qrow = p.q + (long long)(q_start + qi[t]) * p.q_row_stride + (long long)(g * G + hg[t]) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int d0 = ks * 32 + lc * 8;
      qf[t][ks] = (row_ok[t] && d0 < D) ? *(const bf16x8*)(qrow + d0) : zero8;
    }
  }
  // key range of the block and of this wave (rows of a wave are contiguous: 32 of them)
  const int last_row = (M < m0 + BM ? M : m0 + BM) - 1;
  const int kv_end = ctx + last_row / G + 1;
  int kv_begin = 0;
  if (p.window > 0) {
    kv_begin = ctx + m0 / G - p.window + 1;
    if (kv_begin < 0) kv_begin = 0;
  }
  const int wave_first = m0 + wave * RT * 16;
  const int wave_last = (M < wave_first + RT * 16 ? M : wave_first + RT * 16) - 1;
  const bool wave_live = wave_first < M;
  const int wave_kv_end = wave_live ? ctx + wave_last / G + 1 : 0;     // keys >= this are invisible to all rows
  const int wave_min_pos = ctx + wave_first / G;                       // keys <= this are visible to all rows
  int wave_kv_begin = 0, wave_full_begin = 0;                          // window: first visible key of any / of all rows
  if (p.window > 0 && wave_live) {
    wave_kv_begin = wave_min_pos - p.window + 1;
    if (wave_kv_begin < 0) wave_kv_begin = 0;
    wave_full_begin = ctx + wave_last / G - p.window + 1;
    if (wave_full_begin < 0) wave_full_begin = 0;
  }

  // the block's slice of the request's page table goes to LDS once: a tile's loads then hang
  // on one global access, not on two in a row
  // (from the first key of the first TILE, which may lie before kv_begin, to the last key read)
  const int j_first = kv_begin / BN * BN;
  const int first_page = ps.index(j_first);
  const int n_pages = ps.index(kv_end + P - 1) - first_page;
  const bool table_in_lds = n_pages <= TBL_MAX;
  if (table_in_lds)
    for (int i = tid; i < n_pages; i += 256) page_ids[i] = gtable[first_page + i];
  auto page_of = [&](int j) -> long long {
    return table_in_lds ? page_ids[ps.index(j) - first_page] : gtable[ps.index(j)];
  };
  __syncthreads();

  float m_run[RT], l_lane[RT];
  f32x4 acc[RT][NDT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    m_run[t] = -INFINITY;
    l_lane[t] = 0.f;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[t][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // piece c of a V^T tile -> (d, 8-key chunk).  When pages tile the 64 keys (page size 8, 16, 32
  // or 64) consecutive threads walk one page's [D][P] block, which is contiguous in memory;
  // otherwise chunk-major order.
  const bool pages_tile = ps.shift >= 3 && ps.shift <= 6;
  const int cpp_shift = ps.shift - 3;                  // log2(chunks per page row)
  auto v_piece = [&](int c, int& d, int& kc) {
    if (pages_tile) {
      const int q = c >> cpp_shift;                    // (page in tile, d), D rows per page
      const int pg = q / D;
      d = q - pg * D;
      kc = (pg << cpp_shift) + (c & ((1 << cpp_shift) - 1));
    } else {
      d = c / (BN / 8);
      kc = c - d * (BN / 8);
    }
  };
  // ---- global -> registers for one tile; keys at or past kv_end become zeros
  bf16x8 kreg[KPT], vreg[VPT];
  auto fetch = [&](int j0) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int c = tid + i * 256;
      const int key = c / (DK / 8), dc = c - key * (DK / 8);
      const int j = j0 + key;
      bf16x8 v = zero8;
      if (c < KCH && j < kv_end && dc * 8 < D) {
        const long long page = page_of(j);
        v = *(const bf16x8*)(p.k_pages + ((page * p.nkv + g) * P + ps.slot(j)) * (long long)D + dc * 8);
      }
      kreg[i] = v;
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + i * 256;
      int d, kc;
      v_piece(c, d, kc);
      const int j = j0 + kc * 8;
      bf16x8 v = zero8;
      if (c < VCH && j < kv_end) {
        const long long page = page_of(j);
        v = *(const bf16x8*)(p.v_pages + ((page * p.nkv + g) * D + d) * (long long)P + ps.slot(j));
        if (j + 8 > kv_end) {
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (j + e >= kv_end) v[e] = (bf16_t)0.f;
        }
      }
      vreg[i] = v;
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int c = tid + i * 256;
      const int key = c / (DK / 8), dc = c - key * (DK / 8);
      if (c < KCH) *(bf16x8*)(Ks + key * KS_STRIDE + dc * 8) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + i * 256;
      int d, kc;
      v_piece(c, d, kc);
      if (c < VCH) *(bf16x8*)(Vt + d * VT_STRIDE + kc * 8) = vreg[i];
    }
  };

  if (j_first < kv_end) fetch(j_first);
  for (int j0 = j_first; j0 < kv_end; j0 += BN) {
    __syncthreads();          // everyone is done with the previous tile in LDS
    stage();
    __syncthreads();
    if (j0 + BN < kv_end) fetch(j0 + BN);   // in flight while this tile is multiplied

    if (wave_live && j0 < wave_kv_end && j0 + BN > wave_kv_begin) {
      f32x4 s[RT][4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
#pragma unroll
        for (int t = 0; t < RT; ++t) s[t][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks) {
          const bf16x8 a = *(const bf16x8*)(Ks + (kt * 16 + li) * KS_STRIDE + ks * 32 + lc * 8);
#pragma unroll
          for (int t = 0; t < RT; ++t) s[t][kt] = mfma16(a, qf[t][ks], s[t][kt]);
        }
      }
      // interior tile: every key visible to every row of the wave -> no per-element mask
      const bool interior = (j0 + BN - 1 <= wave_min_pos) && (p.window <= 0 || j0 >= wave_full_begin);
#pragma unroll
      for (int t = 0; t < RT; ++t) {
        float tmax = -INFINITY;
        if (interior) {
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float v = s[t][kt][e] * p.scale_log2;
              s[t][kt][e] = v;
              tmax = fmaxf(tmax, v);
            }
        } else {
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int j = j0 + kt * 16 + lc * 4 + e;
              const bool ok = row_ok[t] && j <= pos[t] && (p.window <= 0 || j > pos[t] - p.window);
              const float v = ok ? s[t][kt][e] * p.scale_log2 : -INFINITY;
              s[t][kt][e] = v;
              tmax = fmaxf(tmax, v);
            }
        }
        tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
        tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
        const float m_new = fmaxf(m_run[t], tmax);
        const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
        const float alpha = fast_exp2(m_run[t] - m_use);
        float psum = 0.f;
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float pv = fast_exp2(s[t][kt][e] - m_use);
            s[t][kt][e] = pv;
            psum += pv;
          }
        l_lane[t] = l_lane[t] * alpha + psum;
        m_run[t] = m_new;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) acc[t][dt] *= alpha;
      }
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        bf16x8 b[RT];
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            b[t][e] = (bf16_t)s[t][2 * kk][e];
            b[t][4 + e] = (bf16_t)s[t][2 * kk + 1][e];
          }
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
          const bf16_t* vrow = Vt + (dt * 16 + li) * VT_STRIDE + lc * 4;
          const bf16x4 a0 = *(const bf16x4*)(vrow + (2 * kk) * 16);
          const bf16x4 a1 = *(const bf16x4*)(vrow + (2 * kk + 1) * 16);
          const bf16x8 a = {a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
#pragma unroll
          for (int t = 0; t < RT; ++t) acc[t][dt] = mfma16(a, b[t], acc[t][dt]);
        }
      }
    }
  }

#pragma unroll
  for (int t = 0; t < RT; ++t) {
    float l = l_lane[t] + __shfl_xor(l_lane[t], 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (row_ok[t]) {
      const float inv = 1.f / l;
      bf16_t* o = p.out + (long long)(q_start + qi[t]) * p.nq * D + (long long)(g * G + hg[t]) * D + lc * 4;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        bf16x4 v;
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] = (bf16_t)(acc[t][dt][e] * inv);
        *(bf16x4*)(o + dt * 16) = v;
      }
    }
  }
}

extern "C" int jv_attn_prefill_rows_per_block() { return BM; }

// ------------------------------------------------------------------------------------ decode
constexpr int BND = 32;  // keys per wave iteration

__global__ void __launch_bounds__(256) attn_decode_kernel(AttnArgs p) {
  extern __shared__ float smem[];  // per wave: m[16], l[16], acc[16][D]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lc = lane >> 4;
  const int G = p.nq / p.nkv, P = p.page_size;
  const PageSplit ps{P, p.page_shift};
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
      const long long page = ok ? table[ps.index(j)] : 0;
      const bf16_t* krow = p.k_pages + ((page * p.nkv + g) * P + (ok ? ps.slot(j) : 0)) * (long long)D;
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
      const long long page = ok ? table[ps.index(j)] : 0;
      const bf16_t* vbase = p.v_pages + (page * p.nkv + g) * (long long)D * P + (ok ? ps.slot(j) : 0);
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
static int check_common(AttnArgs& a) {
  if (a.page_size <= 0 || a.page_size % 8 != 0) return (int)hipErrorInvalidValue;
  a.page_shift = -1;
  for (int sft = 3; sft < 31; ++sft)
    if ((1 << sft) == a.page_size) a.page_shift = sft;
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
