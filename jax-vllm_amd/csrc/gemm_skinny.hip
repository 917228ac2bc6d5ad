// y[M,N] = x[M,K] * W[N,K]^T for few rows (M <= 64), bf16 in, float accumulate: the
// weight-streaming matrix product of decode steps, bound by HBM bandwidth.
//
// v_mfma_f32_16x16x32_bf16 with A = 16 rows of W, B = 16 rows of x (both K-contiguous, so
// every lane loads 16 contiguous bytes per operand and nothing is transposed); the
// accumulator holds y^T[n][m].
//
// A block has WR x WK waves: wave (wr, wk) owns W rows [16*(WR*block + wr), +16) and, of
// every K chunk of WK*STEP columns, the slice wk.  W goes from global memory straight into
// MFMA operands, one step ahead of its use.  x must not take that road (it would double
// the vector-memory traffic of a kernel that lives on it): the block copies only the valid
// rows of each x chunk into LDS once, double-buffered, and all its waves read their B
// operands from there.  Partial tiles of the WK slices are added through LDS in a fixed
// order, so a result does not depend on M, on the grid or on timing.
//
// Optional epilogue for the feed-forward's first product: when the rows of W alternate gate and
// up rows, y[m, j] = act(x.W[2j]) * (x.W[2j+1]) straight from the float accumulators (a lane
// holds both numbers of a pair), which saves the activation kernel and its round trip.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define SK_PAD 8  // bf16 elements of padding per LDS row (keeps 16-byte reads of 16 rows off the same banks)

// Up to 16 waves for one tile of x rows (128 registers a lane); at most 8 beyond, where the
// accumulators, the B operands and the x pieces in flight need more.
template <int MT, int NKS, typename OutT, bool PAIRS>
__global__ void __launch_bounds__(MT == 1 ? 1024 : 512)
gemm_skinny_kernel(OutT* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                   int M, int N, int K, long long ldx, long long ldy, int WR, int WK, int act) {
  constexpr int STEP = NKS * 32;
  constexpr int ROWS = MT * 16;
  constexpr int XP = 2 * MT;                 // x pieces a thread keeps in flight
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  const int KCB = WK * STEP;                 // columns of one x chunk
  const int LROW = KCB + SK_PAD;             // LDS row length in elements
  bf16_t* xs = (bf16_t*)smem;                // [2][ROWS][LROW]
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int wave = tid >> 6, lane = tid & 63, li = lane & 15, lc = lane >> 4;
  const int wr = wave % WR, wk = wave / WR;
  const int n = (blockIdx.x * WR + wr) * 16 + li;
  const bool n_ok = n < N;
  const bf16_t* wrow = W + (long long)(n_ok ? n : 0) * K + lc * 8;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int n_iter = (K + KCB - 1) / KCB;

  // rows M..ROWS-1 of both buffers stay zero for the whole kernel
  for (int c = tid; c < 2 * ROWS * LROW / 8; c += nthreads) *(bf16x8*)(xs + c * 8) = zero;
  __syncthreads();

  // chunk `it` of x (valid rows only) -> registers -> LDS buffer
  const int xvecs = M * (KCB / 8);           // 16-byte pieces of one chunk
  auto load_x_piece = [&](int it, int c) -> bf16x8 {
    const int m = c / (KCB / 8), kc = c - m * (KCB / 8);
    const int k = it * KCB + kc * 8;
    if (k >= K) return zero;
    return *(const bf16x8*)(x + (long long)m * ldx + k);
  };
  auto store_x_piece = [&](int buf, int c, bf16x8 v) {
    const int m = c / (KCB / 8), kc = c - m * (KCB / 8);
    *(bf16x8*)(xs + (buf * ROWS + m) * LROW + kc * 8) = v;
  };

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  bf16x8 a_cur[NKS], a_nxt[NKS];
  auto load_w = [&](int it, bf16x8* a) {
    const int k0 = it * KCB + wk * STEP;
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      const int k = k0 + ks * 32 + lc * 8;
      a[ks] = (n_ok && k < K) ? *(const bf16x8*)(wrow + k0 + ks * 32) : zero;
    }
  };
  // prologue: chunk 0 into buffer 0, W of iteration 0
  for (int c = tid; c < xvecs; c += nthreads) store_x_piece(0, c, load_x_piece(0, c));
  load_w(0, a_cur);

  for (int it = 0; it < n_iter; ++it) {
    const bool more = it + 1 < n_iter;
    if (more) load_w(it + 1, a_nxt);
    // next chunk's pieces of this thread: up to XP in flight in registers while this chunk is
    // multiplied; what is beyond (many rows, few threads) is copied after the products
    bf16x8 xr[XP];
    if (more) {
#pragma unroll
      for (int i = 0; i < XP; ++i) {
        const int c = tid + i * nthreads;
        xr[i] = c < xvecs ? load_x_piece(it + 1, c) : zero;
      }
    }
    __syncthreads();  // buffer it&1 is complete; everyone is done reading buffer (it+1)&1
    const bf16_t* xb = xs + ((it & 1) * ROWS) * LROW + wk * STEP + lc * 8;
    // the B operands of one 32-column step are read a step ahead of their products (the fence
    // keeps the compiler from moving each read down to its product, which would then wait a full
    // LDS round trip every time)
    bf16x8 bfr[2][MT];
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) bfr[0][mt] = *(const bf16x8*)(xb + (mt * 16 + li) * LROW);
#pragma unroll
    for (int ks = 0; ks < NKS; ++ks) {
      if (ks + 1 < NKS) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          bfr[(ks + 1) & 1][mt] = *(const bf16x8*)(xb + (mt * 16 + li) * LROW + (ks + 1) * 32);
      }
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_cur[ks], bfr[ks & 1][mt], acc[mt], 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) {
      const int nb = (it + 1) & 1;
#pragma unroll
      for (int i = 0; i < XP; ++i) {
        const int c = tid + i * nthreads;
        if (c < xvecs) store_x_piece(nb, c, xr[i]);
      }
      for (int c = tid + XP * nthreads; c < xvecs; c += nthreads) store_x_piece(nb, c, load_x_piece(it + 1, c));
#pragma unroll
      for (int ks = 0; ks < NKS; ++ks) a_cur[ks] = a_nxt[ks];
    }
  }

  // ---- fixed-order sum over the WK slices; tile of wave (wr, wk), row tile mt, at
  //      red[((wk * WR + wr) * MT + mt) * 256 + lane * 4]
  __syncthreads();  // the x buffers are free now and are reused for the reduction
  float* red = (float*)smem;
  if (WK > 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(f32x4*)(red + (((wk * WR + wr) * MT + mt) * 256 + lane * 4)) = acc[mt];
    __syncthreads();
  }
  // the WK waves of one row tile share its MT column tiles out between them (the loop is
  // unrolled over constant mt: a run-time index would put the accumulators into scratch
  // memory for the whole kernel)
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    if (mt % WK != wk) continue;
    f32x4 s = WK > 1 ? *(const f32x4*)(red + ((wr * MT + mt) * 256 + lane * 4)) : acc[mt];
    for (int w = 1; w < WK; ++w) {
      const f32x4 t = *(const f32x4*)(red + (((w * WR + wr) * MT + mt) * 256 + lane * 4));
      s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
    }
    const int m = mt * 16 + li;
    const int nb = (blockIdx.x * WR + wr) * 16 + lc * 4;
    if (m < M) {
      if (PAIRS) {
        // rows of W alternate gate, up: column pair (2j, 2j+1) -> y[m, j] = act(gate) * up
#pragma unroll
        for (int e = 0; e < 4; e += 2)
          if (nb + e + 1 < N)
            y[(long long)m * ldy + (nb + e) / 2] = from_f32<OutT>(jv_gated(act, s[e], s[e + 1]));
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (nb + e < N) y[(long long)m * ldy + nb + e] = from_f32<OutT>(s[e]);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// Second organisation, for at most 16 rows of x: a block owns one row tile of W, its WK waves
// split K; per phase of up to KP columns every wave first issues ALL its W loads (NL pieces of
// 16 bytes per lane, nothing waits on anything), then the block copies the phase's x columns
// into LDS (MP = 8 or 16 rows; B-operand lanes of rows >= MP read row % MP, their results are
// never stored), one barrier, and the products run as the weights arrive.  One or two barriers
// per phase instead of one per 128 columns.
// K may also be shared out to gridDim.y blocks (k_per columns each, a multiple of KP): block
// (tile, s) then writes the partial product of its columns to y + s * y_part, and whoever reads
// y adds the parts in the order of s.  A narrow matrix gets enough blocks that way to keep the
// memory system busy (a fifth of the chip's bandwidth is lost at 256 blocks against 1,024).
template <int NL, typename OutT>
__global__ void __launch_bounds__(1024)
gemm_skinny_resident_kernel(OutT* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                            int M, int N, int K_all, long long ldx, long long ldy, int WK, int MP, int KP,
                            int k_per, long long y_part) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16_t* xs = (bf16_t*)smem;                // [MP][KP + SK_PAD]
  const int LROW = KP + SK_PAD;
  const int tid = threadIdx.x, nthreads = blockDim.x;
  const int wk = tid >> 6, lane = tid & 63, li = lane & 15, lc = lane >> 4;
  const int n = blockIdx.x * 16 + li;
  const int kb = blockIdx.y * k_per;         // this block's columns are [kb, kb + K)
  const int K = K_all - kb < k_per ? K_all - kb : k_per;
  // no load inside a branch: a row beyond N reads the last row (its outputs are never stored), a piece
  // beyond the block's columns reads the row's last piece again, against zeros in x
  const bf16_t* wrow = W + (long long)min(n, N - 1) * K_all + kb;
  x += kb;
  y += blockIdx.y * y_part;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int SL = NL * 32;                    // columns of one wave per phase; KP == WK * SL
  const int n_phase = (K + KP - 1) / KP;
  // rows M..MP-1 stay zero
  for (int c = tid; c < MP * LROW / 8; c += nthreads) *(bf16x8*)(xs + c * 8) = zero;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  const int xvecs = M * (KP / 8);
  const bf16_t* xrow_lds = xs + (li % MP) * LROW + wk * SL + lc * 8;
  for (int p = 0; p < n_phase; ++p) {
    const int k0 = p * KP + wk * SL;
    bf16x8 a[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) a[i] = *(const bf16x8*)(wrow + min(k0 + i * 32 + lc * 8, K - 8));
    __syncthreads();  // zero fill (first phase) or the previous phase's reads are done
    for (int c = tid; c < xvecs; c += nthreads) {
      const int m = c / (KP / 8), kc = c - m * (KP / 8);
      const int k = p * KP + kc * 8;
      *(bf16x8*)(xs + m * LROW + kc * 8) = k < K ? *(const bf16x8*)(x + (long long)m * ldx + k) : zero;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const bf16x8 b = *(const bf16x8*)(xrow_lds + i * 32);
      acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b, acc, 0, 0, 0);
    }
  }
  __syncthreads();
  float* red = (float*)smem;
  if (WK > 1) {
    *(f32x4*)(red + (wk * 256 + lane * 4)) = acc;
    __syncthreads();
  }
  if (wk == 0) {
    f32x4 s = acc;
    for (int w = 1; w < WK; ++w) {
      const f32x4 t = *(const f32x4*)(red + (w * 256 + lane * 4));
      s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
    }
    const int nb = blockIdx.x * 16 + lc * 4;
    if (li < M) {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (nb + e < N) y[(long long)li * ldy + nb + e] = from_f32<OutT>(s[e]);
    }
  }
}

template <int NL, typename OutT>
static int launch_resident(void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                           long long ldy, int WK, int ksplit, hipStream_t stream) {
  const int MP = M <= 8 ? 8 : 16;
  const int KP = WK * NL * 32;
  // columns per block: the phases shared out evenly, whole phases each
  const int phases = (K + KP - 1) / KP;
  if (ksplit < 1 || ksplit > phases || ksplit > 65535) return (int)hipErrorInvalidValue;
  const int k_per = (phases + ksplit - 1) / ksplit * KP;
  if ((long long)k_per * (ksplit - 1) >= K) return (int)hipErrorInvalidValue;   // a block without columns
  size_t shmem = (size_t)MP * (KP + SK_PAD) * 2;
  if (shmem < (size_t)WK * 256 * 4) shmem = (size_t)WK * 256 * 4;
  if (shmem > 160 * 1024) return (int)hipErrorInvalidValue;
  if (shmem > 64 * 1024) {
    static bool raised = false;
    if (!raised) {
      hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_resident_kernel<NL, OutT>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return (int)e;
      raised = true;
    }
  }
  hipLaunchKernelGGL((gemm_skinny_resident_kernel<NL, OutT>), dim3((N + 15) / 16, ksplit), dim3(WK * 64), shmem,
                     stream, (OutT*)y, (const bf16_t*)x, (const bf16_t*)W, M, N, K, ldx, ldy, WK, MP, KP, k_per,
                     (long long)M * ldy);
  return JV_LAUNCH_CHECK();
}

template <typename OutT>
static int dispatch_resident(int nl, void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                             long long ldy, int WK, int ksplit, hipStream_t s) {
  switch (nl) {
    case 2: return launch_resident<2, OutT>(y, x, W, M, N, K, ldx, ldy, WK, ksplit, s);
    case 4: return launch_resident<4, OutT>(y, x, W, M, N, K, ldx, ldy, WK, ksplit, s);
    case 8: return launch_resident<8, OutT>(y, x, W, M, N, K, ldx, ldy, WK, ksplit, s);
    case 16: return launch_resident<16, OutT>(y, x, W, M, N, K, ldx, ldy, WK, ksplit, s);
  }
  return (int)hipErrorInvalidValue;
}

static size_t skinny_shmem(int MT, int NKS, int WR, int WK) {
  const size_t xbytes = (size_t)2 * MT * 16 * (WK * NKS * 32 + SK_PAD) * 2;
  const size_t rbytes = WK > 1 ? (size_t)WR * WK * MT * 256 * 4 : 0;
  return xbytes > rbytes ? xbytes : rbytes;
}

template <int MT, int NKS, typename OutT, bool PAIRS>
static int launch_skinny(void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                         long long ldy, int WR, int WK, int act, hipStream_t stream) {
  const size_t shmem = skinny_shmem(MT, NKS, WR, WK);
  if (shmem > 64 * 1024) {
    static bool raised = false;  // per instantiation
    if (!raised) {
      hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, NKS, OutT, PAIRS>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return (int)e;
      raised = true;
    }
  }
  const int blocks = (N + 16 * WR - 1) / (16 * WR);
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, NKS, OutT, PAIRS>), dim3(blocks), dim3(WR * WK * 64), shmem,
                     stream, (OutT*)y, (const bf16_t*)x, (const bf16_t*)W, M, N, K, ldx, ldy, WR, WK, act);
  return JV_LAUNCH_CHECK();
}

template <int NKS, typename OutT, bool PAIRS>
static int dispatch_mt(void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                       long long ldy, int WR, int WK, int act, hipStream_t s) {
  switch ((M + 15) / 16) {
    case 1: return launch_skinny<1, NKS, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
    case 2: return launch_skinny<2, NKS, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
    case 3: return launch_skinny<3, NKS, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
    case 4: return launch_skinny<4, NKS, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
  }
  return (int)hipErrorInvalidValue;
}

template <typename OutT, bool PAIRS>
static int dispatch_nks(int nks, void* y, const void* x, const void* W, int M, int N, int K,
                        long long ldx, long long ldy, int WR, int WK, int act, hipStream_t s) {
  switch (nks) {
    case 2: return dispatch_mt<2, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
    case 4: return dispatch_mt<4, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
    case 8: return dispatch_mt<8, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, WR, WK, act, s);
  }
  return (int)hipErrorInvalidValue;
}

// ---------------------------------------------------------------------------------------------
// Third organisation, for at most 16 rows of x (32 with NL <= 8: two row tiles) and an inner size
// of at most 8 * NL * 32: blocks that stay.  Each of a block's 8 waves keeps ITS slice of x (NL steps of 32 columns) in registers
// as MFMA B operands for the whole kernel, so the loop over the block's row tiles of W touches
// LDS only to add the 8 waves' partial tiles: no staging of x, no barrier between the loads.
// The next tile's weights are asked for before the current tile is multiplied and reduced.
// A longer inner size is shared out to gridDim.y groups of blocks, 8 * NL * 32 columns each,
// which write float partial products to y + group * M * ldy (added by the reader, in order).
// Rows of x that come un-normalised from add_parts_unscaled_kernel: output row m is multiplied by
// rsqrt(sum_j ssq[m][j] / width + eps), j < shares, ssq rows of 16 floats (the norm's scale commutes with the
// product; with the inner size shared out every partial product is scaled).  ssq == nullptr: no scale.
struct RowScale {
  const float* ssq;
  int shares;       // at most 16
  float inv_width, eps;
  int act;          // PAIRS: the gate's activation (JV_ACT_*)
};

// No load of the loop sits inside a branch (the compiler would wrap each in a branch of its own, and wait at
// its end): rows of W beyond N read the last row (their outputs are never stored), rows of x beyond M read
// the last row (likewise); EDGE (the inner size is not ksplit * 8 * NL * 32 exactly): columns beyond K read
// the row's last piece again, against zeros in x.
//
// SLOTS > 0 (a divisor of NL): instead of two whole tiles that take turns, W sits in SLOTS slots of NL / SLOTS
// pieces; part q of every tile goes through slot q, which is filled with the next tile's part as soon as it has
// been multiplied, so all slots but one are in flight.  With 4 slots that is three quarters of a tile on its way
// in half the registers of the two-tile scheme: what two row tiles of x with 16 pieces a wave need to fit (128
// registers of x, 64 of W).
template <int NL, int MT, typename OutT, bool PAIRS, bool EDGE, int SLOTS = 0>
__global__ void __launch_bounds__(512)
gemm_skinny_persistent_kernel(OutT* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                              int M, int N, int K, long long ldx, long long ldy, RowScale rs) {
  y += (long long)blockIdx.y * M * ldy;
  // the 8 waves' partial tiles, in two buffers that take turns: one barrier per tile (the waves that do
  // not add may run ahead into the next tile, whose partials go to the other buffer; nobody can be two
  // tiles ahead of the adding wave, which has to pass the barrier in between)
  __shared__ __attribute__((aligned(16))) float red[2][8 * MT * 256];
  const int tid = threadIdx.x;
  const int wk = tid >> 6, lane = tid & 63, li = lane & 15, lc = lane >> 4;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  const int k0 = (blockIdx.y * 8 + wk) * NL * 32 + lc * 8;     // this lane's first column
  const int n_tiles = (N + 15) / 16;
  // x: rows mt * 16 + li (zero beyond M), this wave's columns
  bf16x8 b[MT][NL];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int k = k0 + i * 32, m = min(mt * 16 + li, M - 1);
      const bf16x8 v = *(const bf16x8*)(x + (long long)m * ldx + (EDGE ? min(k, K - 8) : k));
      b[mt][i] = (!EDGE || k < K) ? v : zero;
    }
  // a tile beyond the last (the prefetch after the last tile) reads the first pieces of W, the same for all lanes
  // the scale of this lane's output row (wave mt adds row tile mt): asked for now, used after the first tile;
  // without a scale the loads read x (no load inside a branch) and get no weight
  // (one 16-byte load a lane: the 4 lanes of a row hold its 16 shares; every block reads these few lines,
  // so every instruction more would queue up at one place in the L2)
  f32x4 row_sq;
  {
    const int m = min((wk < MT ? wk : 0) * 16 + li, M - 1);
    const float* sp = rs.ssq ? rs.ssq + (long long)m * 16 + lc * 4 : (const float*)x;
    row_sq = *(const f32x4*)sp;
  }
  // pieces first .. first + CNT - 1 of a tile
  auto load_pieces = [&](int tile, int first, auto& a) {
    constexpr int CNT = sizeof(a) / sizeof(a[0]);
    const int n = min(tile * 16 + li, N - 1);
    const bool real = tile < n_tiles;
    const bf16_t* wrow = W + (real ? (long long)n * K : 0);
    const int kk = (real ? k0 : 0) + first * 32;
#pragma unroll
    for (int i = 0; i < CNT; ++i) a[i] = *(const bf16x8*)(wrow + (EDGE ? min(kk + i * 32, K - 8) : kk + i * 32));
  };
  auto load_tile = [&](int tile, bf16x8 (&a)[NL]) { load_pieces(tile, 0, a); };
  auto multiply_pieces = [&](int first, const auto& a, f32x4 (&acc)[MT]) {
    constexpr int CNT = sizeof(a) / sizeof(a[0]);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < CNT; ++i)
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b[mt][first + i], acc[mt], 0, 0, 0);
  };
  // the 8 waves' sums of a tile, added in fixed order and stored
  auto reduce_store = [&](int tile, const f32x4 (&acc)[MT], int buf) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(f32x4*)(red[buf] + ((wk * MT + mt) * 256 + lane * 4)) = acc[mt];
    __syncthreads();
    if (wk < MT) {                                 // wave mt adds row tile mt, in fixed order: wave 0, 1, ..., 7
      const int mt = wk;
      f32x4 s = *(const f32x4*)(red[buf] + (mt * 256 + lane * 4));
#pragma unroll
      for (int w = 1; w < 8; ++w) {
        const f32x4 t = *(const f32x4*)(red[buf] + ((w * MT + mt) * 256 + lane * 4));
        s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
      }
      const int nb = tile * 16 + lc * 4;           // the accumulator holds y^T[n = lc*4+e][m = mt*16 + li]
      const int m = mt * 16 + li;
      if (rs.ssq) {                                // a fixed order of adding: the same scale in every tile and block
        float sq = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j) sq += lc * 4 + j < rs.shares ? row_sq[j] : 0.f;
        sq += __shfl_xor(sq, 16, 64);
        sq += __shfl_xor(sq, 32, 64);
        const float inv = rsqrtf(sq * rs.inv_width + rs.eps);
        s[0] *= inv; s[1] *= inv; s[2] *= inv; s[3] *= inv;
      }
      if (m < M) {
        if (PAIRS) {
#pragma unroll
          for (int e = 0; e < 4; e += 2)
            if (nb + e + 1 < N)
              y[(long long)m * ldy + (nb + e) / 2] = from_f32<OutT>(jv_gated(rs.act, s[e], s[e + 1]));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (nb + e < N) y[(long long)m * ldy + nb + e] = from_f32<OutT>(s[e]);
        }
      }
    }
  };
  // The next tile's weights are asked for before this tile is multiplied, without a condition (beyond the
  // last tile the last one is read again): after a conditional prefetch the compiler must assume that
  // nothing younger is in flight, and its wait for this tile's first piece then waits for the prefetch too.
  int tile = blockIdx.x;                             // the launch has no more blocks than tiles
  if constexpr (SLOTS == 0) {
    auto finish_tile = [&](int t, bf16x8 (&a)[NL], int buf) {
      f32x4 acc[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
      multiply_pieces(0, a, acc);
      reduce_store(t, acc, buf);
    };
    bf16x8 a0[NL], a1[NL];
    load_tile(tile, a0);
    for (;;) {
      int next = tile + gridDim.x;
      __builtin_amdgcn_sched_barrier(0);
      load_tile(next, a1);
      __builtin_amdgcn_sched_barrier(0);
      finish_tile(tile, a0, 0);
      if (next >= n_tiles) break;
      tile = next;
      next = tile + gridDim.x;
      __builtin_amdgcn_sched_barrier(0);
      load_tile(next, a0);
      __builtin_amdgcn_sched_barrier(0);
      finish_tile(tile, a1, 1);
      if (next >= n_tiles) break;
      tile = next;
    }
  } else {
    static_assert(SLOTS == 0 || NL % (SLOTS ? SLOTS : 1) == 0, "a slot holds a whole number of pieces");
    constexpr int S = NL / (SLOTS ? SLOTS : 1);
    bf16x8 slot[SLOTS ? SLOTS : 1][S];
#pragma unroll
    for (int q = 0; q < SLOTS; ++q) load_pieces(tile, q * S, slot[q]);
    for (int buf = 0;; buf ^= 1) {
      const int next = tile + gridDim.x;
      f32x4 acc[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int q = 0; q < SLOTS; ++q) {
        __builtin_amdgcn_sched_barrier(0);
        multiply_pieces(q * S, slot[q], acc);
        __builtin_amdgcn_sched_barrier(0);
        load_pieces(next, q * S, slot[q]);
      }
      __builtin_amdgcn_sched_barrier(0);
      reduce_store(tile, acc, buf);
      if (next >= n_tiles) break;
      tile = next;
    }
  }
}

template <int NL, int MT, typename OutT, bool PAIRS, int SLOTS = 0>
static int launch_persistent(void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                             long long ldy, int blocks, int ksplit, RowScale rs, hipStream_t stream) {
  const int n_tiles = (N + 15) / 16;
  blocks = (blocks + ksplit - 1) / ksplit;           // per group
  if (blocks > n_tiles) blocks = n_tiles;
  if (K == ksplit * 8 * NL * 32)
    hipLaunchKernelGGL((gemm_skinny_persistent_kernel<NL, MT, OutT, PAIRS, false, SLOTS>), dim3(blocks, ksplit), dim3(512), 0,
                       stream, (OutT*)y, (const bf16_t*)x, (const bf16_t*)W, M, N, K, ldx, ldy, rs);
  else
    hipLaunchKernelGGL((gemm_skinny_persistent_kernel<NL, MT, OutT, PAIRS, true, SLOTS>), dim3(blocks, ksplit), dim3(512), 0,
                       stream, (OutT*)y, (const bf16_t*)x, (const bf16_t*)W, M, N, K, ldx, ldy, rs);
  return JV_LAUNCH_CHECK();
}

// wr == -2: nks = NL in {4, 5, 8, 10, 12, 16, 17, 20}, wk = blocks in all; the inner size must be at most
// ksplit * 8 * NL * 32 and more than (ksplit - 1) * 8 * NL * 32.  Up to 16 rows with every NL, up
// to 32 rows (two row tiles of x in registers) with NL <= 8 and, W in slots, with NL 12 and 16;
// up to 64 rows with NL <= 5.
template <typename OutT, bool PAIRS>
static int dispatch_persistent(int nl, void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                               long long ldy, int blocks, int ksplit, RowScale rs, hipStream_t s) {
  if (M > 64 || (M > 16 && nl > 16) || (M > 32 && nl > 5) || blocks < 1 || ksplit > 65535 ||
      K > (long long)ksplit * 8 * nl * 32 || K <= (long long)(ksplit - 1) * 8 * nl * 32)
    return (int)hipErrorInvalidValue;
  if (M > 48) {
    switch (nl) {
      case 4: return launch_persistent<4, 4, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
      case 5: return launch_persistent<5, 4, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    }
    return (int)hipErrorInvalidValue;
  }
  if (M > 32) {
    switch (nl) {
      case 4: return launch_persistent<4, 3, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
      case 5: return launch_persistent<5, 3, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    }
    return (int)hipErrorInvalidValue;
  }
  if (M > 16) {
    switch (nl) {
      case 4: return launch_persistent<4, 2, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
      case 5: return launch_persistent<5, 2, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
      case 8: return launch_persistent<8, 2, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
      case 12: return launch_persistent<12, 2, OutT, PAIRS, 4>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
      case 16: return launch_persistent<16, 2, OutT, PAIRS, 4>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    }
    return (int)hipErrorInvalidValue;
  }
  switch (nl) {
    case 4: return launch_persistent<4, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 5: return launch_persistent<5, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 8: return launch_persistent<8, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 10: return launch_persistent<10, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 12: return launch_persistent<12, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 16: return launch_persistent<16, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 17: return launch_persistent<17, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
    case 20: return launch_persistent<20, 1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, blocks, ksplit, rs, s);
  }
  return (int)hipErrorInvalidValue;
}

// Shape of the block chosen from the problem.  Measured on MI355X (weights beyond the last-level
// cache): one row tile per block with 8 K slices of 128 columns streams fastest for up to 16
// rows of x at every matrix shape of an 8B-class model; more row tiles per block lose more to
// the wider barrier than they save on x.
static void skinny_config(int M, int N, int K, int* wr, int* wk, int* nks) {
  const int MT = (M + 15) / 16;
  int WR = 1, WK = 8, NKS = 4;
  // LDS: 2 * MT*16 rows * WK*NKS*32 columns * 2 bytes <= 64 KB  ->  MT * WK * NKS <= 32
  while (MT * WK * NKS > 32 && NKS > 2) NKS /= 2;
  while (MT * WK * NKS > 32 && WK > 1) WK /= 2;
  // at least two iterations per wave, or the prefetch has nothing to hide
  while (WK > 1 && K < 2 * WK * NKS * 32) WK /= 2;
  while (NKS > 2 && K < 2 * WK * NKS * 32) NKS /= 2;
  (void)N;
  *wr = WR; *wk = WK; *nks = NKS;
}

// out_f32: 0 -> y is bf16, 1 -> y is float.  x is [M, K] with row stride ldx.
// gate_act: JV_ACT_* (not 0) -> the rows of W alternate gate and up rows and y[m, j] =
//      act(x.W[2j]) * (x.W[2j+1]) is bf16 [M, N/2] (a gated feed-forward's first product with its
//      activation as epilogue).
// wr, wk, nks: block shape (row tiles, K slices, MFMA steps per iteration); 0 picks them.
// wr == -1 selects the resident-x organisation (M <= 16, no activation): wk waves, nks in {2, 4, 8, 16}
// weight pieces per wave and phase.
// ksplit > 1 (resident-x organisation or blocks that stay, float output only): K is shared out to ksplit blocks per
// row tile and y is [ksplit][M][ldy], partial products that the reader adds in that order.
static int gemm_skinny_entry(void* y, const void* x, const void* W, int M, int N, int K, long long ldx, long long ldy,
                             int out_f32, int gate_act, int wr, int wk, int nks, int ksplit, RowScale rs,
                             void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (rs.ssq && (wr != -2 || rs.shares < 1 || rs.shares > 16)) return (int)hipErrorInvalidValue;   // only the staying blocks scale rows
  if (M > 64 || K <= 0 || K % 8 != 0 || ldx % 8 != 0) return (int)hipErrorInvalidValue;
  if (gate_act && (!jv_act_known(gate_act) || out_f32 || N % 2 != 0 || wr == -1)) return (int)hipErrorInvalidValue;
  rs.act = gate_act;
  if (ksplit < 1 || (ksplit > 1 && ((wr != -1 && wr != -2) || !out_f32))) return (int)hipErrorInvalidValue;
  if (wr == -2) {   // blocks that stay: wk = number of blocks, nks = weight pieces per wave
    hipStream_t s = (hipStream_t)stream;
    if (gate_act) return dispatch_persistent<bf16_t, true>(nks, y, x, W, M, N, K, ldx, ldy, wk, ksplit, rs, s);
    return out_f32 ? dispatch_persistent<float, false>(nks, y, x, W, M, N, K, ldx, ldy, wk, ksplit, rs, s)
                   : dispatch_persistent<bf16_t, false>(nks, y, x, W, M, N, K, ldx, ldy, wk, ksplit, rs, s);
  }
  if (wr == -1) {
    if (M > 16 || wk < 1 || wk > 16) return (int)hipErrorInvalidValue;
    hipStream_t s = (hipStream_t)stream;
    return out_f32 ? dispatch_resident<float>(nks, y, x, W, M, N, K, ldx, ldy, wk, ksplit, s)
                   : dispatch_resident<bf16_t>(nks, y, x, W, M, N, K, ldx, ldy, wk, ksplit, s);
  }
  if (wr == 0 && wk == 0 && nks == 0 && M <= 2 && !gate_act && K >= 2048 && K <= 4096 && N >= 8192) {
    // one or two rows against a wide matrix: the resident-x organisation measured ~10 % faster
    hipStream_t s = (hipStream_t)stream;
    return out_f32 ? dispatch_resident<float>(16, y, x, W, M, N, K, ldx, ldy, 8, 1, s)
                   : dispatch_resident<bf16_t>(16, y, x, W, M, N, K, ldx, ldy, 8, 1, s);
  }
  int cwr, cwk, cnks;
  skinny_config(M, N, K, &cwr, &cwk, &cnks);
  if (wr <= 0) wr = cwr;
  if (wk <= 0) wk = cwk;
  if (nks <= 0) nks = cnks;
  const int MT = (M + 15) / 16;
  if (wr * wk > (MT == 1 ? 16 : 8) || (nks != 2 && nks != 4 && nks != 8)) return (int)hipErrorInvalidValue;
  if (skinny_shmem(MT, nks, wr, wk) > 160 * 1024) return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  if (gate_act) return dispatch_nks<bf16_t, true>(nks, y, x, W, M, N, K, ldx, ldy, wr, wk, gate_act, s);
  if (out_f32) return dispatch_nks<float, false>(nks, y, x, W, M, N, K, ldx, ldy, wr, wk, 0, s);
  return dispatch_nks<bf16_t, false>(nks, y, x, W, M, N, K, ldx, ldy, wr, wk, 0, s);
}

extern "C" int jv_gemm_skinny_bf16(void* y, const void* x, const void* W, int M, int N, int K,
                                   long long ldx, long long ldy, int out_f32, int gate_act, int wr,
                                   int wk, int nks, int ksplit, void* stream) {
  return gemm_skinny_entry(y, x, W, M, N, K, ldx, ldy, out_f32, gate_act, wr, wk, nks, ksplit,
                           RowScale{nullptr, 0, 0.f, 0.f, 0}, stream);
}

// The same for rows of x that add_parts_unscaled left un-normalised (blocks that stay only, wr == -2):
// output row m is multiplied by rsqrt(sum_{j < shares} ssq[m * 16 + j] / width + eps).
extern "C" int jv_gemm_skinny_scaled_bf16(void* y, const void* x, const void* W, int M, int N, int K,
                                          long long ldx, long long ldy, int out_f32, int gate_act, int wr,
                                          int wk, int nks, int ksplit, const float* ssq, int shares, int width,
                                          float eps, void* stream) {
  if (!ssq || width <= 0) return (int)hipErrorInvalidValue;
  return gemm_skinny_entry(y, x, W, M, N, K, ldx, ldy, out_f32, gate_act, wr, wk, nks, ksplit,
                           RowScale{ssq, shares, 1.f / (float)width, eps, 0}, stream);
}
