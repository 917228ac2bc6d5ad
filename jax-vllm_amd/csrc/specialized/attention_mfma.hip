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
//                   in LDS and shared by the 4 waves; causal limit and window per row.  Head sizes that are
//                   multiples of 32 up to 128 have a kernel of their own instead (32x32x16 products, one tile
//                   of 32 rows per wave, tiles straight from global memory into LDS): see JV_PREFILL32.
//   decode kernel:  one query per request; each of the 4 waves streams its own 32-key tiles
//                   straight from global memory into MFMA operands (no LDS), the waves'
//                   partial (max, sum, acc) are merged in LDS; with num_splits > 1 several
//                   blocks share a request's keys and a second kernel merges their partials.
#include "../common.h"
#include <type_traits>

#ifndef JV_HEAD_DIM
#error "compile with -DJV_HEAD_DIM=<head size>"
#endif
static_assert(JV_HEAD_DIM % 16 == 0 && JV_HEAD_DIM >= 16 && JV_HEAD_DIM <= 256, "head size");
#if JV_HEAD_DIM % 32 == 0 && JV_HEAD_DIM <= 128
#define JV_PREFILL32 1   // the prefill kernel with 32-row tiles is built, the one with 16-row tiles is not
#endif

constexpr int D = JV_HEAD_DIM;
constexpr int NDT = D / 16;                // 16-wide tiles of the head dimension (output)
constexpr int DK = (D + 31) / 32 * 32;     // head dimension padded to the QK contraction step
constexpr int NKS = DK / 32;
constexpr int BN = 64;                     // keys per LDS tile (prefill)
constexpr int KS_STRIDE = DK + 16;         // bf16 elements per key row in LDS: with a row stride of 8 dwords mod 16,
                                           // 16-byte reads of 16 rows run at the full LDS rate (measured)
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
  const int* work;            // prefill: [n_work][3] = (request, first row of group 0, first row of group 1 or -1); decode: [n_work] = request
  int page_size, page_shift, nq, nkv;   // page_shift: log2(page_size) or -1
  float scale_log2;           // softmax scale * log2(e)
  int window;                 // <= 0: none
  // decode only
  int num_splits;
  float* part_acc;            // [n_work, nq, num_splits, D]
  float* part_ml;             // [n_work, nq, num_splits, 2] (max, sum)
};

// ------------------------------------------------------------------------------------ prefill
// A block of 4 waves works on one or two GROUPS of 64 rows of one request and one kv head: wave w
// takes rows 16w..16w+15 of each group (two groups for head sizes up to 128, one above: registers).
// The host pairs a group that sees many keys with one that sees few, so that all blocks and all
// waves have about the same number of (row tile, key tile) products; where both groups see a key
// tile, every K fragment and V^T fragment read from LDS feeds both.  K/V tiles of 64 keys go
// global -> registers while the previous tile is multiplied, and registers -> LDS between two
// barriers.  Keys are masked only on tiles that cross a row's causal limit or window edge.
constexpr int RT = D <= 128 ? 2 : 1;       // row groups per block = row tiles per wave
constexpr int GROUP_ROWS = 64;             // 4 waves x 16 rows
constexpr float RESCALE_STEP = 8.f;        // growth of a row's maximum (powers of two) that moves its reference: p <= 2^8
constexpr int KCH = BN * (DK / 8);         // 16-byte pieces of a K tile
constexpr int VCH = D * (BN / 8);          // 16-byte pieces of a V^T tile
constexpr int KPT = (KCH + 255) / 256;     // pieces per thread
constexpr int VPT = (VCH + 255) / 256;
constexpr int TBL_MAX = 2048;              // page-table entries a block keeps in LDS at a time
constexpr int NO_GAP = 0x7fffffff;

#if JV_HEAD_DIM <= 128
#define PREFILL_OCCUPANCY __attribute__((amdgpu_waves_per_eu(2, 2)))  // two waves per SIMD (both kernels): one wave computes while the other waits
#else
#define PREFILL_OCCUPANCY
#endif
#ifndef JV_PREFILL32
// PAGES: 1 = the page size is 8, 16, 32 or 64 (pages tile the 64 keys: a thread's slot in its
// page is the same in every tile), 2 = a larger power of two, 0 = any other multiple of 8.
template <int PAGES>
__global__ void __launch_bounds__(256) PREFILL_OCCUPANCY attn_prefill_kernel(AttnArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[BN * KS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t Vt[D * VT_STRIDE];
  __shared__ int page_ids[TBL_MAX];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lc = lane >> 4;
  // consecutive blocks take the kv heads of one work item: with the heaviest items first the whole
  // grid is heaviest-first, and (blocks going round the chip's 8 dies) a kv head's keys stay in
  // the L2 of nkv/8 dies, or of one
  const int g = blockIdx.x % p.nkv, item = blockIdx.x / p.nkv;
  const int r = p.work[3 * item];
  const int G = p.nq / p.nkv, P = p.page_size;
  const PageSplit ps{P, PAGES == 0 ? -1 : p.page_shift};
  const int q_start = p.cu_seqlens[r], q_len = p.cu_seqlens[r + 1] - q_start;
  const int ctx = p.context_lens[r];
  const int M = q_len * G;
  const int* gtable = p.block_tables + (long long)r * p.table_stride;
  const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};

  // this lane's rows (one per group), and per group the key ranges of the block and of the wave
  int qi[RT], hg[RT], pos[RT];
  bool row_ok[RT];
  bf16x8 qf[RT][NKS];
  int blk_begin[RT], blk_end[RT];          // keys [begin, end) some row of the block's group sees; empty if no group
  bool wave_live[RT];
  int wave_kv_begin[RT], wave_kv_end[RT];  // keys some row of the wave's tile sees
  int wave_full_begin[RT], wave_min_pos[RT];  // keys in [full_begin, min_pos] are seen by every row of the tile
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int m0 = p.work[3 * item + 1 + t];       // first row of the group, or -1
    const int row = m0 + wave * 16 + li;
    row_ok[t] = m0 >= 0 && row < M;
    qi[t] = row_ok[t] ? row / G : 0;
    hg[t] = row_ok[t] ? row - qi[t] * G : 0;
    pos[t] = ctx + qi[t];
    const bf16_t* qrow = p.q + (long long)(q_start + qi[t]) * p.q_row_stride + (long long)(g * G + hg[t]) * D;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int d0 = ks * 32 + lc * 8;
      qf[t][ks] = (row_ok[t] && d0 < D) ? *(const bf16x8*)(qrow + d0) : zero8;
    }
    blk_begin[t] = blk_end[t] = 0;
    if (m0 >= 0 && m0 < M) {
      const int last_row = (M < m0 + GROUP_ROWS ? M : m0 + GROUP_ROWS) - 1;
      blk_end[t] = ctx + last_row / G + 1;
      if (p.window > 0) {
        blk_begin[t] = ctx + m0 / G - p.window + 1;
        if (blk_begin[t] < 0) blk_begin[t] = 0;
      }
    }
    const int wave_first = m0 + wave * 16;
    wave_live[t] = m0 >= 0 && wave_first < M;
    const int wave_last = (M < wave_first + 16 ? M : wave_first + 16) - 1;
    wave_kv_end[t] = wave_live[t] ? ctx + wave_last / G + 1 : 0;
    wave_min_pos[t] = ctx + wave_first / G;
    wave_kv_begin[t] = wave_full_begin[t] = 0;
    if (p.window > 0 && wave_live[t]) {
      wave_kv_begin[t] = wave_min_pos[t] - p.window + 1;
      if (wave_kv_begin[t] < 0) wave_kv_begin[t] = 0;
      wave_full_begin[t] = ctx + wave_last / G - p.window + 1;
      if (wave_full_begin[t] < 0) wave_full_begin[t] = 0;
    }
  }
  // The tiles the block walks: those of the one range, or of the union of the two; when a window
  // leaves a gap between them the walk jumps from gap_from to gap_to (both multiples of BN).
  int j_first, kv_end, gap_from = NO_GAP, gap_to = NO_GAP;
  {
    int b0 = blk_begin[0] / BN * BN, e0 = blk_end[0];
    int b1 = b0, e1 = 0;
    if (RT > 1) { b1 = blk_begin[RT - 1] / BN * BN; e1 = blk_end[RT - 1]; }
    if (e1 <= b1) { b1 = b0; e1 = e0; }             // no second group
    if (e0 <= b0) { b0 = b1; e0 = e1; }             // no first group
    if (b1 < b0) { int x = b0; b0 = b1; b1 = x; x = e0; e0 = e1; e1 = x; }
    j_first = b0;
    kv_end = e0 > e1 ? e0 : e1;
    const int e0_up = (e0 + BN - 1) / BN * BN;
    if (b1 > e0_up) { gap_from = e0_up; gap_to = b1; }
  }
  auto next_tile = [&](int j0) { return j0 + BN == gap_from ? gap_to : j0 + BN; };
  if (kv_end <= j_first) return;                    // nothing to do (the same in every thread)

  // A slice of the request's page table sits in LDS: a tile's loads then hang on one global
  // access, not on two in a row.  It starts at the page of the first key of the first tile and
  // is moved forward when a tile reaches past its end.
  const int last_page = ps.index(kv_end - 1);
  int seg_first = 0;
  auto load_table = [&](int j) {        // called by all threads, between barriers
    seg_first = ps.index(j);
    int n = last_page - seg_first + 1;
    if (n > TBL_MAX) n = TBL_MAX;
    for (int i = tid; i < n; i += 256) page_ids[i] = gtable[seg_first + i];
  };
  load_table(j_first);
  __syncthreads();

  float m_run[RT], m_ref[RT], l_lane[RT];
  f32x4 acc[RT][NDT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    m_run[t] = -INFINITY;
    m_ref[t] = -INFINITY;
    l_lane[t] = 0.f;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) acc[t][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // piece c of a V^T tile -> (d, 8-key chunk).  When pages tile the 64 keys consecutive threads
  // walk one page's [D][P] block, which is contiguous in memory; otherwise chunk-major order.
  const int cpp_shift = ps.shift - 3;                  // PAGES == 1: log2(chunks per page row)
  auto v_piece = [&](int c, int& d, int& kc) {
    if (PAGES == 1) {
      const int q = c >> cpp_shift;                    // (page in tile, d), D rows per page
      const int pg = q / D;
      d = q - pg * D;
      kc = (pg << cpp_shift) + (c & ((1 << cpp_shift) - 1));
    } else {
      d = c / (BN / 8);
      kc = c - d * (BN / 8);
    }
  };
  // ---- global -> registers for one tile.  Nothing here looks at a loaded value or branches per
  // lane, so the loads stay in flight while the previous tile is multiplied.  A piece past the
  // last key reads the same slot of the last page (allocated memory, masked later by position),
  // and what must be zero is made zero when the registers are written to LDS.
  const unsigned page_stride = (unsigned)p.nkv * (unsigned)P * (unsigned)D;   // elements; the host checks it fits
  // per-thread constants of the pieces: the element offset inside a page; a piece's first key in
  // the tile is recomputed where it is needed (registers are scarce here)
  auto k_piece_key = [&](int i) {
    int c = tid + i * 256;
    if (KCH % 256 != 0 && c > KCH - 1) c = KCH - 1;
    return c / (DK / 8);
  };
  auto v_piece_key = [&](int i) {
    int c = tid + i * 256;
    if (VCH % 256 != 0 && c > VCH - 1) c = VCH - 1;
    int d, kc;
    v_piece(c, d, kc);
    return kc * 8;
  };
  int k_off[KPT], v_off[VPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    int c = tid + i * 256;
    if (KCH % 256 != 0 && c > KCH - 1) c = KCH - 1;
    const int key = c / (DK / 8);
    int dc = c - key * (DK / 8);
    if (DK != D && dc * 8 >= D) dc = 0;
    k_off[i] = (g * P + (PAGES == 1 ? (key & (P - 1)) : 0)) * D + dc * 8;
  }
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    int c = tid + i * 256;
    if (VCH % 256 != 0 && c > VCH - 1) c = VCH - 1;
    int d, kc;
    v_piece(c, d, kc);
    v_off[i] = (g * D + d) * P + (PAGES == 1 ? ((kc * 8) & (P - 1)) : 0);
  }
  bf16x8 kreg[KPT], vreg[VPT];
  auto fetch = [&](int j0) {
    int j_hi = j0 + BN - 1;
    if (j_hi > kv_end - 1) j_hi = kv_end - 1;
    if (ps.index(j_hi) - seg_first >= TBL_MAX) {   // same decision in every thread
      __syncthreads();
      load_table(j0);
      __syncthreads();
    }
    const int tile_page = ps.index(j0) - seg_first, end_page = last_page - seg_first;
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      int pi, off = k_off[i];
      if (PAGES == 1) {
        pi = tile_page + (k_piece_key(i) >> ps.shift);
      } else {
        const int j = j0 + k_piece_key(i);
        pi = ps.index(j) - seg_first;
        off += ps.slot(j) * D;
      }
      if (pi > end_page) pi = end_page;
      const unsigned page = (unsigned)page_ids[pi];
      kreg[i] = *(const bf16x8*)(p.k_pages + ((unsigned long long)page * page_stride + (unsigned)off));
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      int pi, off = v_off[i];
      if (PAGES == 1) {
        pi = tile_page + (v_piece_key(i) >> ps.shift);
      } else {
        const int j = j0 + v_piece_key(i);
        pi = ps.index(j) - seg_first;
        off += ps.slot(j);
      }
      if (pi > end_page) pi = end_page;
      const unsigned page = (unsigned)page_ids[pi];
      vreg[i] = *(const bf16x8*)(p.v_pages + ((unsigned long long)page * page_stride + (unsigned)off));
    }
  };
  // ---- registers -> LDS.  K columns that pad the head size and V entries of keys at or past
  // kv_end become zeros (their probabilities are zeros, and zero times a stale NaN is not).
  auto stage = [&](int j0) {
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int c = tid + i * 256;
      const int key = c / (DK / 8), dc = c - key * (DK / 8);
      bf16x8 v = kreg[i];
      if (DK != D && dc * 8 >= D) v = zero8;
      if (KCH % 256 == 0 || c < KCH) *(bf16x8*)(Ks + key * KS_STRIDE + dc * 8) = v;
    }
    const bool last_tile = j0 + BN > kv_end;      // the same in every thread
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int c = tid + i * 256;
      int d, kc;
      v_piece(c, d, kc);
      bf16x8 v = vreg[i];
      if (last_tile) {
        const int j = j0 + kc * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (j + e >= kv_end) v[e] = (bf16_t)0.f;
      }
      if (VCH % 256 == 0 || c < VCH) *(bf16x8*)(Vt + d * VT_STRIDE + kc * 8) = v;
    }
  };

  // ---- one key tile times the row tiles named by MASK (bit t: the wave's tile of group t).
  // LDS fragments are read one group ahead of the products that use them (K: the 4 key tiles of one
  // 32-wide slice of the head; V^T: 2 head tiles of one 32-key half); the scheduling fences keep
  // the compiler from moving a group's reads down to their first use, where every product would
  // wait a full LDS round trip.
  constexpr int VG = 2;                                  // head tiles per V^T fragment group
  constexpr int GPK = (NDT + VG - 1) / VG;               // groups per 32-key half
  auto read_k = [&](bf16x8 (&f)[4], int ks) {
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) f[kt] = *(const bf16x8*)(Ks + (kt * 16 + li) * KS_STRIDE + ks * 32 + lc * 8);
  };
  auto read_v = [&](bf16x8 (&f)[VG], int q) {
    const int kk = q / GPK, d0 = (q - kk * GPK) * VG;
#pragma unroll
    for (int i = 0; i < VG; ++i) {
      if (d0 + i < NDT) {
        const bf16_t* vrow = Vt + ((d0 + i) * 16 + li) * VT_STRIDE + lc * 4;
        const bf16x4 a0 = *(const bf16x4*)(vrow + (2 * kk) * 16);
        const bf16x4 a1 = *(const bf16x4*)(vrow + (2 * kk + 1) * 16);
        f[i] = bf16x8{a0[0], a0[1], a0[2], a0[3], a1[0], a1[1], a1[2], a1[3]};
      }
    }
  };
  auto multiply = [&](auto mask_const, int j0) {
    constexpr int MASK = decltype(mask_const)::value;
    f32x4 s[RT][4];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) s[t][kt] = f32x4{0.f, 0.f, 0.f, 0.f};
    bf16x8 kf[2][4];
    read_k(kf[0], 0);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks + 1 < NKS) read_k(kf[(ks + 1) & 1], ks + 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int t = 0; t < RT; ++t)
          if ((MASK >> t) & 1) s[t][kt] = mfma16(kf[ks & 1][kt], qf[t][ks], s[t][kt]);
      __builtin_amdgcn_sched_barrier(0);
    }
    bf16x8 vf[2][VG];
    read_v(vf[0], 0);                    // on its way during the softmax
    __builtin_amdgcn_sched_barrier(0);
    bf16x8 pb[2][RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      if (!((MASK >> t) & 1)) continue;
      // interior tile: every key visible to every row of the tile -> no per-element mask
      const bool interior = (j0 + BN - 1 <= wave_min_pos[t]) && (p.window <= 0 || j0 >= wave_full_begin[t]);
      float tmax = -INFINITY;
      // the maximum is taken over raw scores (the scale is positive); the scale enters in the
      // exponent's multiply-add: p = exp2(s * scale_log2 - m * scale_log2)
      if (interior) {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e) tmax = fmaxf(tmax, s[t][kt][e]);
      } else {
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int j = j0 + kt * 16 + lc * 4 + e;
            const bool ok = row_ok[t] && j <= pos[t] && (p.window <= 0 || j > pos[t] - p.window);
            const float v = ok ? s[t][kt][e] : -INFINITY;
            s[t][kt][e] = v;
            tmax = fmaxf(tmax, v);
          }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run[t], tmax);                       // raw-score units
      m_run[t] = m_new;
      // The exponents are taken against m_ref, which follows the running maximum only when that
      // has grown by more than RESCALE_STEP (in powers of two): sums and outputs are then brought
      // to the new reference.  Most tiles change no row's reference and skip that work; a row's
      // numbers do not depend on the other rows of its wave, only the skipping does.
      const bool grown = (m_new - m_ref[t]) * p.scale_log2 > RESCALE_STEP;   // false while no key is visible
      if (__builtin_amdgcn_ballot_w64(grown) != 0) {
        const float alpha = grown ? fast_exp2((m_ref[t] - m_new) * p.scale_log2) : 1.f;   // 0 from -inf
        if (grown) m_ref[t] = m_new;
        l_lane[t] *= alpha;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) acc[t][dt] *= alpha;
      }
      const float m_use = (m_ref[t] == -INFINITY) ? 0.f : m_ref[t] * p.scale_log2;
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const float pv = fast_exp2(fmaf(s[t][kt][e], p.scale_log2, -m_use));
          s[t][kt][e] = pv;
          psum += pv;
        }
      l_lane[t] += psum;
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          pb[kk][t][e] = (bf16_t)s[t][2 * kk][e];
          pb[kk][t][4 + e] = (bf16_t)s[t][2 * kk + 1][e];
        }
    }
#pragma unroll
    for (int q = 0; q < 2 * GPK; ++q) {
      if (q + 1 < 2 * GPK) read_v(vf[(q + 1) & 1], q + 1);
      __builtin_amdgcn_sched_barrier(0);
      const int kk = q / GPK, d0 = (q - kk * GPK) * VG;
#pragma unroll
      for (int i = 0; i < VG; ++i)
#pragma unroll
        for (int t = 0; t < RT; ++t)
          if (d0 + i < NDT && ((MASK >> t) & 1)) acc[t][d0 + i] = mfma16(vf[q & 1][i], pb[kk][t], acc[t][d0 + i]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  fetch(j_first);
  for (int j0 = j_first; j0 < kv_end;) {
    const int j_next = next_tile(j0);
    stage(j0);
    __syncthreads();
    if (j_next < kv_end) fetch(j_next);        // in flight while this tile is multiplied
    int mask = 0;
#pragma unroll
    for (int t = 0; t < RT; ++t)
      if (wave_live[t] && j0 < wave_kv_end[t] && j0 + BN > wave_kv_begin[t]) mask |= 1 << t;
    if (RT > 1 && mask == 3) multiply(std::integral_constant<int, 3>{}, j0);
    else if (RT > 1 && mask == 2) multiply(std::integral_constant<int, 2>{}, j0);
    else if (mask == 1) multiply(std::integral_constant<int, 1>{}, j0);
    __syncthreads();
    j0 = j_next;
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

#endif  // !JV_PREFILL32

// ------------------------------------------------------------------------------------ prefill, 32-row tiles
// Head sizes that are multiples of 32 up to 128 take this kernel.  It reads the same work items
// (two groups of 64 rows) but gives every wave ONE tile of 32 rows (waves 0, 1: first group,
// waves 2, 3: second group) and multiplies with v_mfma_f32_32x32x16_bf16: a 16-byte fragment of K
// or V^T read from LDS then feeds a product of 32 cycles, twice as much as with 16x16x32 tiles
// of a single row tile, and the kernel lives on the LDS rate (128 B/clk for 16-byte reads, half
// of that for 8-byte ones).  What makes every LDS access one of 16 bytes:
//   * S^T accumulators of a 32-key block hold, for the lane halves h = 0, 1, product rows
//     8i + 4h + j (i, j < 4).  Product row 8i + 4h + j is fed with key 16(i/2) + 8h + 4(i%2) + j of
//     the block (only a lane's LDS read address changes), so the two accumulator quads i = 2s,
//     2s + 1 of a lane are the 8 CONSECUTIVE keys 16s + 8h .. + 7: exactly the B operand of
//     O^T += V^T P^T for keys 16s .. 16s + 15, whose A operand is then a plain 16-byte read of
//     V^T[d][16s + 8h ..].
//   * both tiles are stored in 16-byte chunks whose position inside each 256-byte line is
//     xor-ed with the line number: reads of 32 rows at one column and writes of whole rows are
//     both conflict-free (measured).
// Tiles are double-buffered in LDS: one barrier per 64 keys.  With pages of 16 keys and a head size
// that is a power of two (PAGES == 16) a wave also overlaps its own work: the scores of tile i + 1 are
// multiplied while the probabilities of tile i are made (measured at 32 q heads over 8 kv heads of
// 128: 2,048 tokens 58 against 63 us, 8,192 tokens 566 against 638, 512 tokens after 16,000: 306
// against 383; the kernel then keeps the matrix unit busy 55..60 % of the time at the 1.9 GHz it
// runs at, the LDS about as much, and neither can be filled further by two waves a SIMD).
#ifdef JV_PREFILL32
typedef float f32x16 __attribute__((ext_vector_type(16)));
// a wave in a burst of products goes first: the other wave of its SIMD (of the compute unit's other block) then
// does its softmax meanwhile instead of contending for the matrix unit
#define JV_PRIO(x) __builtin_amdgcn_s_setprio(x)
__device__ __forceinline__ f32x16 mfma32(bf16x8 a, bf16x8 b, f32x16 c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
}
constexpr int NQS = D / 16;                // contraction steps of S^T = K Q^T
constexpr int NDB = D / 32;                // 32-row blocks of O^T
constexpr int CPK = D / 8;                 // 16-byte chunks of a key row
constexpr int TBL32 = 1024;                // page-table entries a block keeps in LDS at a time
constexpr int PCS = BN * CPK / 256;        // 16-byte pieces of a K tile (and of a V^T tile) per thread
constexpr bool KB_ADDS = (32 * CPK / 16) % 16 == 0;   // the second key block's chunks are the first's plus a constant
__device__ __forceinline__ int swizzle(int q) { return q ^ ((q >> 4) & 15); }   // chunk index -> chunk position

template <int PAGES>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) attn_prefill32_kernel(AttnArgs p) {
  __shared__ __attribute__((aligned(16))) bf16_t Ks[2][BN * D];
  __shared__ __attribute__((aligned(16))) bf16_t Vs[2][D * BN];
  // FAST: pages of 16 keys and a head size that is a power of two.  Every load instruction of a wave
  // then lies in ONE page, whose number is a scalar read straight from the request's table, and a
  // lane's address is that page's base plus a constant of the lane.
  constexpr bool FAST = PAGES == 16;
  static_assert(!FAST || (64 % CPK == 0), "the fast path needs whole keys per load instruction");
  __shared__ int page_ids[FAST ? 1 : TBL32];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // a scalar: branches on it are uniform
  const int l32 = lane & 31, h = lane >> 5;
  const int g = blockIdx.x % p.nkv, item = blockIdx.x / p.nkv;
  const int r = p.work[3 * item];
  const int G = p.nq / p.nkv, P = FAST ? 16 : p.page_size;
  const PageSplit ps{P, PAGES == 0 ? -1 : (FAST ? 4 : p.page_shift)};
  const int q_start = p.cu_seqlens[r], q_len = p.cu_seqlens[r + 1] - q_start;
  const int ctx = p.context_lens[r];
  const int M = q_len * G;
  const int* gtable = p.block_tables + (long long)r * p.table_stride;

  // ---- the block's two groups: keys [begin, end) that some row of a group sees
  int blk_begin[2], blk_end[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int m0 = p.work[3 * item + 1 + t];
    blk_begin[t] = blk_end[t] = 0;
    if (m0 >= 0 && m0 < M) {
      const int last_row = (M < m0 + 64 ? M : m0 + 64) - 1;
      blk_end[t] = ctx + last_row / G + 1;
      if (p.window > 0) {
        blk_begin[t] = ctx + m0 / G - p.window + 1;
        if (blk_begin[t] < 0) blk_begin[t] = 0;
      }
    }
  }
  // ---- this wave's tile of 32 rows and this lane's row
  const int m0 = p.work[3 * item + 1 + (wave >> 1)];
  const int wave_first = m0 + (wave & 1) * 32;
  const bool wave_live = m0 >= 0 && wave_first < M;
  const int wave_last = (M < wave_first + 32 ? M : wave_first + 32) - 1;
  const int wave_kv_end = wave_live ? ctx + wave_last / G + 1 : 0;
  const int wave_min_pos = ctx + wave_first / G;
  int wave_kv_begin = 0, wave_full_begin = 0;
  if (p.window > 0 && wave_live) {
    wave_kv_begin = wave_min_pos - p.window + 1;
    if (wave_kv_begin < 0) wave_kv_begin = 0;
    wave_full_begin = ctx + wave_last / G - p.window + 1;
    if (wave_full_begin < 0) wave_full_begin = 0;
  }
  const int row = wave_first + l32;
  const bool row_ok = wave_live && row < M;
  const int qi = row_ok ? row / G : 0, hg = row_ok ? row - qi * G : 0;
  const int pos = ctx + qi;
  bf16x8 qf[NQS];                          // B operand: row l32, head elements 16 ks + 8 h .. + 7
  {
    const bf16_t* qrow = p.q + (long long)(q_start + qi) * p.q_row_stride + (long long)(g * G + hg) * D + h * 8;
    const bf16x8 zero8 = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int ks = 0; ks < NQS; ++ks) qf[ks] = row_ok ? *(const bf16x8*)(qrow + ks * 16) : zero8;
  }

  // ---- the tiles the block walks (the union of the two groups' ranges; a window may leave a gap)
  int j_first, kv_end, gap_from = NO_GAP, gap_to = NO_GAP;
  {
    int b0 = blk_begin[0] / BN * BN, e0 = blk_end[0];
    int b1 = blk_begin[1] / BN * BN, e1 = blk_end[1];
    if (e1 <= b1) { b1 = b0; e1 = e0; }
    if (e0 <= b0) { b0 = b1; e0 = e1; }
    if (b1 < b0) { int x = b0; b0 = b1; b1 = x; x = e0; e0 = e1; e1 = x; }
    j_first = b0;
    kv_end = e0 > e1 ? e0 : e1;
    const int e0_up = (e0 + BN - 1) / BN * BN;
    if (b1 > e0_up) { gap_from = e0_up; gap_to = b1; }
  }
  auto next_tile = [&](int j0) { return j0 + BN == gap_from ? gap_to : j0 + BN; };
  if (kv_end <= j_first) return;                    // nothing to do (the same in every thread)

  const int last_page = ps.index(kv_end - 1);
  int seg_first = 0;
  auto load_table = [&](int j) {                    // called by all threads, between barriers
    seg_first = ps.index(j);
    int n = last_page - seg_first + 1;
    if (n > TBL32) n = TBL32;
    for (int i = tid; i < n; i += 256) page_ids[i] = gtable[seg_first + i];
  };
  if (!FAST) {
    load_table(j_first);
    __syncthreads();
  }

  // ---- pieces of a tile.  A tile goes from global memory straight into LDS (no registers between):
  // instruction i of wave w fills the 64 chunk positions (4i + w) * 64 .. + 63 of the buffer, lane l the
  // position (4i + w) * 64 + l, so the lane asks for the chunk that belongs there (both swizzles are
  // their own inverses).  K is stored key by key, 256-byte lines xor-ed with the line number.  V^T is
  // stored d row by d row of 64 keys in the general path; in the fast path page by page, [page][d][2
  // chunks], positions xor-ed with the lowest bit of the line number: a wave's 64 chunks are then 32
  // whole d rows of one page, 1 KB in one piece, and the reads of 32 d at one key chunk stay
  // conflict-free (8 d rows a line, neighbouring lines swap their even and odd positions).
  const unsigned page_stride = (unsigned)p.nkv * (unsigned)P * (unsigned)D;   // elements; the host checks it fits
  auto v_swizzle = [&](int q) { return FAST ? (q ^ ((q >> 4) & 1)) : swizzle(q); };
  int k_off[PCS], v_off[PCS], k_key[PCS], v_key[PCS];
#pragma unroll
  for (int i = 0; i < PCS; ++i) {
    const int pos = (4 * i + wave) * 64 + lane;
    const int q = swizzle(pos);
    const int key = q / CPK, dc = q - key * CPK;
    k_key[i] = key;
    k_off[i] = (g * P + (PAGES != 0 && PAGES != 2 ? (key & (P - 1)) : 0)) * D + dc * 8;
    const int qv = v_swizzle(pos);
    if (FAST) {
      const int pg = qv / (2 * D), d = (qv - pg * 2 * D) >> 1, c = qv & 1;
      v_key[i] = pg * 16 + c * 8;
      v_off[i] = (g * D + d) * 16 + c * 8;
    } else {
      const int d = qv / (BN / 8), kc = qv - d * (BN / 8);
      v_key[i] = kc * 8;
      v_off[i] = (g * D + d) * P + (PAGES == 1 ? ((kc * 8) & (P - 1)) : 0);
    }
  }
  // 16 bytes a lane from global memory straight into LDS: lane l of the wave writes to `lds` + 16 l.  Written
  // in assembly on purpose: told that a vector-memory instruction writes LDS, the compiler waits for ALL
  // such loads in flight before every LDS read it cannot prove to be elsewhere (it cannot tell the two
  // buffers apart), which is exactly the overlap this kernel is built on.  The waits are ours: arrived()
  // before the barrier that hands a buffer over.
  typedef const bf16_t* gptr_t;
  typedef const bf16_t* lptr_t;
  auto dma16 = [&](gptr_t src, lptr_t lds) {
    const unsigned at = (unsigned)(unsigned long long)(const __attribute__((address_space(3))) void*)lds;
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(at) : "memory", "m0");
  };
  // Nothing here looks at a loaded value.  A piece past the last key reads the same slot of the last
  // page (allocated memory): K there is masked by position, V is zeroed in LDS by fix_tail.
  // fast path: the PCS pages of this wave's instructions for the tile at j0, as scalars from the
  // table (read-only for the kernel's life, hence the constant address space: scalar loads that
  // nothing else waits on).  They are asked for one tile before the tile's loads are issued.
  typedef const __attribute__((address_space(4))) int* ctable_t;
  const ctable_t ctable = (ctable_t)(unsigned long long)gtable;
  auto pages_of = [&](int j0, unsigned (&pg)[PCS]) {
#pragma unroll
    for (int i = 0; i < PCS; ++i) {
      int pi = (j0 >> 4) + (((4 * i + wave) * 64) / (2 * D));   // first key of the instruction, (4i + w) * 64 / CPK, over 16
      if (pi > last_page) pi = last_page;
      pg[i] = (unsigned)ctable[pi];
    }
  };
  auto fetch = [&](int j0, int b) {
    int j_hi = j0 + BN - 1;
    if (j_hi > kv_end - 1) j_hi = kv_end - 1;
    if (ps.index(j_hi) - seg_first >= TBL32) {      // same decision in every thread
      __syncthreads();
      load_table(j0);
      __syncthreads();
    }
    const int tile_page = ps.index(j0) - seg_first, end_page = last_page - seg_first;
#pragma unroll
    for (int i = 0; i < PCS; ++i) {
      int pi, off = k_off[i];
      if (PAGES == 1) {
        pi = tile_page + (k_key[i] >> ps.shift);
      } else {
        const int j = j0 + k_key[i];
        pi = ps.index(j) - seg_first;
        off += ps.slot(j) * D;
      }
      if (pi > end_page) pi = end_page;
      const unsigned page = (unsigned)page_ids[pi];
      dma16(p.k_pages + ((unsigned long long)page * page_stride + (unsigned)off),
              &Ks[b][(4 * i + wave) * 64 * 8]);
    }
#pragma unroll
    for (int i = 0; i < PCS; ++i) {
      int pi, off = v_off[i];
      if (PAGES == 1) {
        pi = tile_page + (v_key[i] >> ps.shift);
      } else {
        const int j = j0 + v_key[i];
        pi = ps.index(j) - seg_first;
        off += ps.slot(j);
      }
      if (pi > end_page) pi = end_page;
      const unsigned page = (unsigned)page_ids[pi];
      dma16(p.v_pages + ((unsigned long long)page * page_stride + (unsigned)off),
              &Vs[b][(4 * i + wave) * 64 * 8]);
    }
  };
  // V entries of keys at or past kv_end become zeros (their probabilities are zeros, and zero times a
  // stale NaN is not): every thread cleans the pieces it asked for, once they have arrived.
  auto fix_tail = [&](int j0, int b) {
#pragma unroll
    for (int i = 0; i < PCS; ++i) {
      const int j = j0 + v_key[i];
      if (j + 8 > kv_end) {
        bf16x8* at = (bf16x8*)&Vs[b][((4 * i + wave) * 64 + lane) * 8];
        bf16x8 v = *at;
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (j + e >= kv_end) v[e] = (bf16_t)0.f;
        *at = v;
      }
    }
  };
  auto arrived = [&]() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); };

  // ---- LDS read addresses (elements).  K: product row l32 = 8i + 4hh + j reads key 16(i/2) + 8hh + 4(i%2) + j.
  const int krow = ((l32 >> 4) << 4) | (((l32 >> 2) & 1) << 3) | (((l32 >> 3) & 1) << 2) | (l32 & 3);
  auto k_read = [&](int kb, int ks) { return swizzle((kb * 32 + krow) * CPK + 2 * ks + h) * 8; };
  int kr[NQS];
#pragma unroll
  for (int ks = 0; ks < NQS; ++ks) kr[ks] = k_read(0, ks);
  int vr[BN / 16];                                  // d = l32 (+ 32 db: adds a constant), keys 16 s + 8 h .. + 7
#pragma unroll
  for (int s = 0; s < BN / 16; ++s)
    vr[s] = (FAST ? v_swizzle(s * 2 * D + l32 * 2 + h) : swizzle(l32 * (BN / 8) + 2 * s + h)) * 8;
  constexpr int V_DB = FAST ? 32 * 2 * 8 : 32 * BN;  // elements from one block of 32 d to the next
  // the key that element e = 4i + j of a 32-key block's accumulator belongs to, less the block's first
  auto acc_key = [&](int e) { return 16 * (e >> 3) + 8 * h + 4 * ((e >> 2) & 1) + (e & 3); };

  float m_run = -INFINITY, m_ref = -INFINITY, l_lane = 0.f;
  f32x16 acc[NDB];
#pragma unroll
  for (int db = 0; db < NDB; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;

  auto multiply = [&](int j0, int b) {
    const bf16_t* Kb = Ks[b];
    const bf16_t* Vb = Vs[b];
    f32x16 s[2];
#pragma unroll
    for (int kb = 0; kb < 2; ++kb)
#pragma unroll
      for (int e = 0; e < 16; ++e) s[kb][e] = 0.f;
    // S^T: fragments are read two steps ahead of their products
    bf16x8 kf[3][2];
    auto read_k = [&](int ks, bf16x8 (&f)[2]) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
        f[kb] = *(const bf16x8*)(Kb + (KB_ADDS ? kr[ks] + kb * 32 * D : k_read(kb, ks)));
    };
    read_k(0, kf[0]);
    if (NQS > 1) read_k(1, kf[1]);
    JV_PRIO(1);
#pragma unroll
    for (int ks = 0; ks < NQS; ++ks) {
      if (ks + 2 < NQS) read_k(ks + 2, kf[(ks + 2) % 3]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) s[kb] = mfma32(kf[ks % 3][kb], qf[ks], s[kb]);
      __builtin_amdgcn_sched_barrier(0);
    }
    JV_PRIO(0);
    bf16x8 vf[2][NDB];
    auto read_v = [&](int sidx, bf16x8 (&f)[NDB]) {
#pragma unroll
      for (int db = 0; db < NDB; ++db) f[db] = *(const bf16x8*)(Vb + vr[sidx] + db * V_DB);
    };
    read_v(0, vf[0]);                    // on its way during the softmax
    __builtin_amdgcn_sched_barrier(0);
    // interior tile: every key visible to every row of the tile -> no per-element mask
    const bool interior = (j0 + BN - 1 <= wave_min_pos) && (p.window <= 0 || j0 >= wave_full_begin);
    float tmax = -INFINITY;
    if (interior) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, s[kb][e]);
    } else {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const int j = j0 + kb * 32 + acc_key(e);
          const bool ok = row_ok && j <= pos && (p.window <= 0 || j > pos - p.window);
          const float v = ok ? s[kb][e] : -INFINITY;
          s[kb][e] = v;
          tmax = fmaxf(tmax, v);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float m_new = fmaxf(m_run, tmax);                          // raw-score units
    m_run = m_new;
    // exponents are taken against m_ref, which follows the running maximum only when that has grown
    // by more than RESCALE_STEP powers of two; most tiles then skip rescaling sums and outputs
    const bool grown = (m_new - m_ref) * p.scale_log2 > RESCALE_STEP;   // false while no key is visible
    if (__builtin_amdgcn_ballot_w64(grown) != 0) {
      const float alpha = grown ? fast_exp2((m_ref - m_new) * p.scale_log2) : 1.f;   // 0 from -inf
      if (grown) m_ref = m_new;
      l_lane *= alpha;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[db][e] *= alpha;
    }
    const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref * p.scale_log2;
    float psum = 0.f;
    bf16x8 pb[BN / 16];                  // P^T operands: keys 16 s + 8 h .. + 7 = elements 8 (s % 2) .. + 7 of block s / 2
#pragma unroll
    for (int sidx = 0; sidx < BN / 16; ++sidx)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pv = fast_exp2(fmaf(s[sidx >> 1][8 * (sidx & 1) + e], p.scale_log2, -m_use));
        psum += pv;
        pb[sidx][e] = (bf16_t)pv;
      }
    l_lane += psum;
    JV_PRIO(1);
#pragma unroll
    for (int sidx = 0; sidx < BN / 16; ++sidx) {
      if (sidx + 1 < BN / 16) read_v(sidx + 1, vf[(sidx + 1) & 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int db = 0; db < NDB; ++db) acc[db] = mfma32(vf[sidx & 1][db], pb[sidx], acc[db]);
      __builtin_amdgcn_sched_barrier(0);
    }
    JV_PRIO(0);
  };

  if constexpr (FAST) {
    // ---- the same walk with a wave's products and its softmax overlapped: while the probabilities of tile i
    // are made (float units), the scores of tile i + 1 are already multiplied (matrix unit), and the first
    // products of O^T += V^T P^T start as soon as their 16 keys' probabilities exist.  K is therefore
    // fetched two tiles ahead and V one: K(i+2) goes where K(i) was, V(i+1) where V(i-1) was.
    auto fetch_k = [&](int b, const unsigned (&pgs)[PCS]) {
#pragma unroll
      for (int i = 0; i < PCS; ++i)
        dma16(p.k_pages + (unsigned long long)pgs[i] * page_stride + (unsigned)k_off[i],
              &Ks[b][(4 * i + wave) * 64 * 8]);
    };
    auto fetch_v = [&](int b, const unsigned (&pgs)[PCS]) {
#pragma unroll
      for (int i = 0; i < PCS; ++i)
        dma16(p.v_pages + (unsigned long long)pgs[i] * page_stride + (unsigned)v_off[i],
              &Vs[b][(4 * i + wave) * 64 * 8]);
    };
    auto read_k = [&](const bf16_t* Kb, int ks, bf16x8 (&f)[2]) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) f[kb] = *(const bf16x8*)(Kb + (KB_ADDS ? kr[ks] + kb * 32 * D : k_read(kb, ks)));
    };
    auto read_v = [&](const bf16_t* Vb, int sidx, bf16x8 (&f)[NDB]) {
#pragma unroll
      for (int db = 0; db < NDB; ++db) f[db] = *(const bf16x8*)(Vb + vr[sidx] + db * V_DB);
    };
    auto qk_step = [&](f32x16 (&sn)[2], const bf16x8 (&f)[2], int ks) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) sn[kb] = mfma32(f[kb], qf[ks], sn[kb]);
    };
    auto pv_step = [&](const bf16x8 (&f)[NDB], const bf16x8& pbs) {
#pragma unroll
      for (int db = 0; db < NDB; ++db) acc[db] = mfma32(f[db], pbs, acc[db]);
    };
    // the row's maximum over the tile, the new reference if it has grown; returns whether any row of the wave moved
    auto row_max = [&](f32x16 (&sc)[2], int j0, float& alpha) -> bool {
      const bool interior = (j0 + BN - 1 <= wave_min_pos) && (p.window <= 0 || j0 >= wave_full_begin);
      float tmax = -INFINITY;
      if (interior) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) tmax = fmaxf(tmax, sc[kb][e]);
      } else {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int j = j0 + kb * 32 + acc_key(e);
            const bool ok = row_ok && j <= pos && (p.window <= 0 || j > pos - p.window);
            const float v = ok ? sc[kb][e] : -INFINITY;
            sc[kb][e] = v;
            tmax = fmaxf(tmax, v);
          }
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float m_new = fmaxf(m_run, tmax);
      m_run = m_new;
      const bool grown = (m_new - m_ref) * p.scale_log2 > RESCALE_STEP;
      alpha = grown ? fast_exp2((m_ref - m_new) * p.scale_log2) : 1.f;
      if (grown) m_ref = m_new;
      return __builtin_amdgcn_ballot_w64(grown) != 0;
    };
    auto rescale = [&](float alpha) {
      l_lane *= alpha;
#pragma unroll
      for (int db = 0; db < NDB; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[db][e] *= alpha;
    };
    auto exp_chunk = [&](const f32x16 (&sc)[2], int sidx, float m_use, bf16x8& pbs) {
      float psum = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pv = fast_exp2(fmaf(sc[sidx >> 1][8 * (sidx & 1) + e], p.scale_log2, -m_use));
        psum += pv;
        pbs[e] = (bf16_t)pv;
      }
      l_lane += psum;
    };
    constexpr int NPS = BN / 16;                       // products O^T += V^T P^T of 16 keys each
    // scores of the next tile only (the wave sees nothing of this one)
    auto tile_qk = [&](f32x16 (&sn)[2], const bf16_t* Kb) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) sn[kb][e] = 0.f;
      bf16x8 kf[2][2];
      read_k(Kb, 0, kf[0]);
#pragma unroll
      for (int ks = 0; ks < NQS; ++ks) {
        if (ks + 1 < NQS) read_k(Kb, ks + 1, kf[(ks + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        qk_step(sn, kf[ks & 1], ks);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // softmax and output products of this tile only
    auto tile_sm = [&](f32x16 (&sc)[2], int j0, const bf16_t* Vb) {
      bf16x8 vf[2][NDB], pb[NPS];
      read_v(Vb, 0, vf[0]);
      float alpha;
      if (row_max(sc, j0, alpha)) rescale(alpha);
      const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref * p.scale_log2;
#pragma unroll
      for (int sidx = 0; sidx < NPS; ++sidx) exp_chunk(sc, sidx, m_use, pb[sidx]);
#pragma unroll
      for (int sidx = 0; sidx < NPS; ++sidx) {
        if (sidx + 1 < NPS) read_v(Vb, sidx + 1, vf[(sidx + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        pv_step(vf[sidx & 1], pb[sidx]);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // both: scores of the next tile under the softmax of this one
    auto tile_both = [&](f32x16 (&sc)[2], f32x16 (&sn)[2], int j0, const bf16_t* Kb, const bf16_t* Vb) {
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) sn[kb][e] = 0.f;
      constexpr int SPG = (NQS + 3) / 4;               // score steps per group (4 groups, one per 16 keys of probabilities)
      bf16x8 kf[2][SPG][2], vf[2][NDB], pb[NPS];
      auto read_group = [&](int gidx, bf16x8 (&f)[SPG][2]) {
#pragma unroll
        for (int i = 0; i < SPG; ++i)
          if (gidx * SPG + i < NQS) read_k(Kb, gidx * SPG + i, f[i]);
      };
      auto qk_group = [&](int gidx, const bf16x8 (&f)[SPG][2]) {
#pragma unroll
        for (int i = 0; i < SPG; ++i)
          if (gidx * SPG + i < NQS) qk_step(sn, f[i], gidx * SPG + i);
      };
      read_group(0, kf[0]);
      // group 0: first score steps under the row maximum
      read_group(1, kf[1]);
      __builtin_amdgcn_sched_barrier(0);
      JV_PRIO(1);
      qk_group(0, kf[0]);
      float alpha;
      const bool moved = row_max(sc, j0, alpha);
      __builtin_amdgcn_sched_barrier(0);
      if (moved) rescale(alpha);
      const float m_use = (m_ref == -INFINITY) ? 0.f : m_ref * p.scale_log2;
      // groups 1..3: score steps under the exponentials of keys 0..47
#pragma unroll
      for (int gidx = 1; gidx < 4; ++gidx) {
        if (gidx + 1 < 4) read_group(gidx + 1, kf[(gidx + 1) & 1]);
        else read_v(Vb, 0, vf[0]);
        __builtin_amdgcn_sched_barrier(0);
        qk_group(gidx, kf[gidx & 1]);
        exp_chunk(sc, gidx - 1, m_use, pb[gidx - 1]);
        __builtin_amdgcn_sched_barrier(0);
      }
      // the first output products under the last exponentials
      read_v(Vb, 1, vf[1]);
      __builtin_amdgcn_sched_barrier(0);
      pv_step(vf[0], pb[0]);
      exp_chunk(sc, NPS - 1, m_use, pb[NPS - 1]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int sidx = 1; sidx < NPS; ++sidx) {
        if (sidx + 1 < NPS) read_v(Vb, sidx + 1, vf[(sidx + 1) & 1]);
        __builtin_amdgcn_sched_barrier(0);
        pv_step(vf[sidx & 1], pb[sidx]);
        __builtin_amdgcn_sched_barrier(0);
      }
      JV_PRIO(0);
    };

    // Every live wave takes every tile the block walks (a tile it sees nothing of is masked like any
    // other: at most one per block when neighbouring groups are paired): one path through the loop.
    f32x16 sa[2], sb[2];
    int j0 = j_first, j1 = next_tile(j0), j2 = j1 < kv_end ? next_tile(j1) : j1;
    unsigned pga[PCS], pgb[PCS];
    pages_of(j0, pga);
    fetch_k(0, pga);
    fetch_v(0, pga);
    if (j1 < kv_end) {
      pages_of(j1, pga);
      fetch_k(1, pga);                                // pga: the pages of tile 1, whose V is fetched in the first turn
    }
    if (j2 < kv_end) pages_of(j2, pgb);
    arrived();
    if (j0 + BN > kv_end) fix_tail(j0, 0);
    __syncthreads();
    if (wave_live) tile_qk(sa, Ks[0]);
    // one turn: tile t (scores in sc, K and V in buffers b), tile t + 1 (scores into sn, K in buffer b ^ 1)
    auto turn = [&](f32x16 (&sc)[2], f32x16 (&sn)[2], int b) {
      const bool has2 = j2 < kv_end;
      fetch_v(b ^ 1, pga);                            // V(t+1) where V(t-1) was
      if (has2) fetch_k(b, pgb);                      // K(t+2) where K(t) was: its scores were made in the last turn
      const int j3 = has2 ? next_tile(j2) : j2;
#pragma unroll
      for (int i = 0; i < PCS; ++i) pga[i] = pgb[i];
      if (j3 < kv_end) pages_of(j3, pgb);
      if (wave_live) tile_both(sc, sn, j0, Ks[b ^ 1], Vs[b]);
      arrived();
      if (j1 + BN > kv_end) fix_tail(j1, b ^ 1);
      __syncthreads();
      j0 = j1; j1 = j2; j2 = j3;
    };
    int b = 0;
    while (j1 < kv_end) {
      turn(sa, sb, 0);
      b = 1;
      if (j1 >= kv_end) break;
      turn(sb, sa, 1);
      b = 0;
    }
    if (wave_live) {                                  // the last tile: nothing follows it
      if (b == 0) tile_sm(sa, j0, Vs[0]);
      else tile_sm(sb, j0, Vs[1]);
    }
  } else {
    fetch(j_first, 0);
    arrived();
    if (j_first + BN > kv_end) fix_tail(j_first, 0);
    __syncthreads();
    int b = 0;
    for (int j0 = j_first; j0 < kv_end;) {
      const int j_next = next_tile(j0);
      const bool more = j_next < kv_end;
      if (more) fetch(j_next, b ^ 1);                 // in flight while this tile is multiplied; nobody reads that
                                                      // buffer: its tile was finished before the last barrier
      if (wave_live && j0 < wave_kv_end && j0 + BN > wave_kv_begin) multiply(j0, b);
      arrived();
      if (more && j_next + BN > kv_end) fix_tail(j_next, b ^ 1);   // own pieces only: no barrier needed before
      __syncthreads();
      j0 = j_next;
      b ^= 1;
    }
  }

  float l = l_lane + __shfl_xor(l_lane, 32, 64);
  if (row_ok) {
    const float inv = 1.f / l;
    bf16_t* o = p.out + (long long)(q_start + qi) * p.nq * D + (long long)(g * G + hg) * D + h * 4;
#pragma unroll
    for (int db = 0; db < NDB; ++db)
#pragma unroll
      for (int i = 0; i < 4; ++i) {                 // accumulator rows 8i + 4h + j of block db
        bf16x4 v;
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] = (bf16_t)(acc[db][4 * i + j] * inv);
        *(bf16x4*)(o + db * 32 + i * 8) = v;
      }
  }
}
#endif

// the host's plan: rows per group, and groups a work item may name
extern "C" int jv_attn_prefill_group_rows() { return GROUP_ROWS; }
extern "C" int jv_attn_prefill_groups_per_item() { return RT; }
// 1: each group of a work item has waves of its own (pair groups that see the same keys); 0: every wave
// takes rows of both groups (pair a light group with a heavy one)
#ifdef JV_PREFILL32
extern "C" int jv_attn_prefill_waves_split() { return 1; }
#else
extern "C" int jv_attn_prefill_waves_split() { return 0; }
#endif

// ------------------------------------------------------------------------------------ decode
constexpr int BND = 32;  // keys per wave iteration
constexpr int DEC_TBL_MAX = 4096;  // page-table entries of a request that a decode block keeps in LDS

__global__ void __launch_bounds__(256) PREFILL_OCCUPANCY attn_decode_kernel(AttnArgs p) {
  extern __shared__ float smem[];  // per wave: m[16], l[16], acc[16][D]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int li = lane & 15, lc = lane >> 4;
  const int G = p.nq / p.nkv, P = p.page_size;
  const PageSplit ps{P, p.page_shift};
  const int mt_per_head = (G + 15) / 16;
  const int w = blockIdx.x;
  // Without a work list the requests are 0, 1, ... and request r's token is row r (a step of
  // decoded tokens only): nothing has to be looked up before the loads below can start.  The
  // kernel's time at small batches is its chain of dependent memory round trips (~1.5 us each
  // for data the previous kernel wrote), so the request's page table row is copied to LDS at
  // once, beside the load of its context length, instead of being read key range by key range
  // after it.
  const int r = p.work ? p.work[w] : w;
  const int g = blockIdx.y / mt_per_head, mt = blockIdx.y - g * mt_per_head;
  const int split = blockIdx.z;
  const int* gtable = p.block_tables + (long long)r * p.table_stride;
  // A table row beyond DEC_TBL_MAX entries does not fit: the block then copies only the entries of its own
  // split's keys, once it knows them (one more round trip, at contexts where that does not matter; the
  // entry point makes sure that a split's entries fit).  Pages are always looked up in LDS: a lookup in
  // global memory beside it would be a load inside a branch, at whose end the compiler waits for every
  // load in flight, tile after tile.
  int* tbl = (int*)(smem + 4 * (32 + 16 * D));
  const bool whole_row = p.table_stride <= DEC_TBL_MAX;
  if (whole_row)
    for (int i = tid; i < p.table_stride; i += 256) tbl[i] = gtable[i];
  const int tok = p.cu_seqlens ? p.cu_seqlens[r] : r;
  const int pos = p.context_lens[r];      // the query's position; keys 0..pos are stored
  const int kv_len = pos + 1;
  int kv_begin = 0;
  if (p.window > 0 && pos - p.window + 1 > 0) kv_begin = pos - p.window + 1;

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

  int tbl_first = 0;                      // table entry that tbl[0] holds
  if (!whole_row && t_lo < t_hi) {
    tbl_first = ps.index(t_lo * BND);
    const int j_last = (t_hi * BND < kv_len ? t_hi * BND : kv_len) - 1;
    int n = ps.index(j_last) - tbl_first + 1;
    if (n > DEC_TBL_MAX) n = DEC_TBL_MAX;             // never, by the entry point's check
    for (int i = tid; i < n; i += 256) tbl[i] = gtable[tbl_first + i];
  }
  __syncthreads();   // the table entries are in LDS
  auto page_at = [&](int idx) -> long long { return tbl[idx - tbl_first]; };
  // One tile's operands, global -> registers.  Nothing here looks at a loaded value, so a tile's
  // loads are in flight while the tile before it is multiplied.  Keys at or past kv_len read the
  // null page: their scores are masked by position, their V entries are zeroed before use.
  //   K operand: lane (key li of sub-tile kt, chunk lc) <- 8 consecutive d of that key
  //   V^T operand: lane (d = dt*16 + li, chunk lc) <- keys kt*16 + lc*4 .. +4 of that d
  // `real` false (the prefetch behind the wave's last tile): everything is read from the null page.  The
  // prefetch is never skipped: after a conditional one the compiler must assume that nothing younger is
  // in flight, and its waits for this tile's operands would wait for the prefetched tile as well.
  auto load_tile = [&](int t, bool real, bf16x8 (&kf)[2][NKS], bf16x4 (&vf)[2][NDT]) {
    const int j0 = t * BND;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int j = j0 + kt * 16 + li;
      const bool ok = real && j < kv_len;
      const long long looked = page_at(ok ? ps.index(j) : tbl_first);
      const long long page = ok ? looked : 0;
      const bf16_t* krow = p.k_pages + ((page * p.nkv + g) * P + (ok ? ps.slot(j) : 0)) * (long long)D;
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) {
        const int d0 = ks * 32 + lc * 8;
        kf[kt][ks] = *(const bf16x8*)(krow + (DK != D && d0 >= D ? 0 : d0));
      }
    }
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      const int j = j0 + kt * 16 + lc * 4;
      const bool ok = real && j < kv_len;
      const long long looked = page_at(ok ? ps.index(j) : tbl_first);
      const long long page = ok ? looked : 0;
      const bf16_t* vbase = p.v_pages + (page * p.nkv + g) * (long long)D * P + (ok ? ps.slot(j) : 0);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) vf[kt][dt] = *(const bf16x4*)(vbase + (long long)(dt * 16 + li) * P);
    }
  };
  auto multiply = [&](int t, bf16x8 (&kf)[2][NKS], bf16x4 (&vf)[2][NDT]) {
    const int j0 = t * BND;
    if (DK != D) {                       // columns that pad the head size to the contraction step
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int ks = 0; ks < NKS; ++ks)
          if (ks * 32 + lc * 8 >= D) kf[kt][ks] = bf16x8{0, 0, 0, 0, 0, 0, 0, 0};
    }
    if (j0 + BND > kv_len) {             // the last tile (the same in every lane): zero times a stale NaN is not zero
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (j0 + kt * 16 + lc * 4 + e >= kv_len) vf[kt][dt][e] = (bf16_t)0.f;
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
  };
  // two register sets take turns: while one tile is multiplied the wave's next one is on its way
  {
    bf16x8 kf_a[2][NKS], kf_b[2][NKS];
    bf16x4 vf_a[2][NDT], vf_b[2][NDT];
    int t = t_lo + wave;
    load_tile(t, t < t_hi, kf_a, vf_a);
    while (t < t_hi) {
      __builtin_amdgcn_sched_barrier(0);
      load_tile(t + 4, t + 4 < t_hi, kf_b, vf_b);
      __builtin_amdgcn_sched_barrier(0);
      multiply(t, kf_a, vf_a);
      t += 4;
      if (t >= t_hi) break;
      __builtin_amdgcn_sched_barrier(0);
      load_tile(t + 4, t + 4 < t_hi, kf_a, vf_a);
      __builtin_amdgcn_sched_barrier(0);
      multiply(t, kf_b, vf_b);
      t += 4;
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
  // All loads of a batch of 8 splits are issued before anything is computed from them: this
  // kernel's time is its chain of dependent memory round trips, not its arithmetic.
  const int w = blockIdx.x, head = blockIdx.y, d = threadIdx.x < D ? threadIdx.x : D - 1;
  const int r = p.work ? p.work[w] : w;
  const int tok = p.cu_seqlens ? p.cu_seqlens[r] : r;
  const long long base = ((long long)w * p.nq + head) * p.num_splits;
  const float2* ml = (const float2*)p.part_ml + base;      // (max, sum) per split
  const float* pa = p.part_acc + base * D + d;
  float mx = -INFINITY, num = 0.f, den = 0.f;
  for (int s0 = 0; s0 < p.num_splits; s0 += 8) {
    float2 v[8];
    float a[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int s = s0 + i < p.num_splits ? s0 + i : p.num_splits - 1;   // a repeat, given no weight below
      v[i] = ml[s];
      a[i] = pa[(long long)s * D];
    }
    float bm = mx;
#pragma unroll
    for (int i = 0; i < 8; ++i) bm = fmaxf(bm, v[i].x);
    if (bm == -INFINITY) continue;                          // nothing stored in these splits or before
    const float keep = fast_exp2(mx - bm);                  // 0 when mx is still -inf
    num *= keep;
    den *= keep;
    mx = bm;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // an empty split (max -inf) may hold anything in its accumulator: it gets no weight and is not read into the sum
      const bool live = s0 + i < p.num_splits && v[i].x != -INFINITY;
      const float f = live ? fast_exp2(v[i].x - mx) : 0.f;
      num += live ? a[i] * f : 0.f;
      den += live ? v[i].y * f : 0.f;
    }
  }
  if (threadIdx.x < D) p.out[(long long)tok * p.nq * D + (long long)head * D + d] = (bf16_t)(num / den);
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
extern "C" int jv_attn_decode_table_entries() { return DEC_TBL_MAX; }
extern "C" int jv_attn_decode_tile_keys() { return BND; }

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
  if ((long long)nkv * page_size * D >= (1ll << 31)) return (int)hipErrorInvalidValue;   // offsets inside a page are 32-bit
  if ((long long)n_work * nkv >= (1ll << 31)) return (int)hipErrorInvalidValue;
  const int mode = (a.page_shift >= 3 && a.page_shift <= 6) ? 1 : (a.page_shift > 6 ? 2 : 0);
#ifdef JV_PREFILL32
  constexpr bool pow2 = (D & (D - 1)) == 0;
  void (*kernel)(AttnArgs) = (page_size == 16 && pow2) ? attn_prefill32_kernel<pow2 ? 16 : 1>
                             : mode == 1 ? attn_prefill32_kernel<1>
                             : mode == 2 ? attn_prefill32_kernel<2> : attn_prefill32_kernel<0>;
#else
  void (*kernel)(AttnArgs) = mode == 1 ? attn_prefill_kernel<1> : (mode == 2 ? attn_prefill_kernel<2> : attn_prefill_kernel<0>);
#endif
  hipLaunchKernelGGL(kernel, dim3(n_work * nkv), dim3(256), 0, (hipStream_t)stream, a);
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
  // a table row that does not fit in LDS whole: every split's own entries must (keys of a split span at most
  // ceil(tiles / splits) tiles of BND keys, hence that many keys over the page size, plus the pages it cuts)
  if (table_stride > DEC_TBL_MAX) {
    const long long tiles = ((long long)table_stride * page_size + BND - 1) / BND;
    const long long per_split = (tiles + a.num_splits - 1) / a.num_splits;
    if (per_split * BND / page_size + 2 > DEC_TBL_MAX) return (int)hipErrorInvalidValue;
  }
  const size_t shmem = 4 * (32 + 16 * D) * sizeof(float) +
                       (size_t)(table_stride <= DEC_TBL_MAX ? table_stride : DEC_TBL_MAX) * sizeof(int);
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
