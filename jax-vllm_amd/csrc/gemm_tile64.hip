// y[M,N] = x[M,K] * W[N,K]^T for 17..64 rows, bf16 in, float accumulate: the matrix product of
// decode steps with many requests.  It is still bound by the weight stream (W is read once, every
// element feeds up to 64 rows), but x no longer fits beside it for free: with 16-row tiles of W
// every tile would pull the whole of x through the caches again, four times the bytes of W at 64
// rows.  So a block takes 64 rows of W (x traffic = the bytes of W at most) and the inner size is
// shared out to `ksplit` blocks per tile so that enough blocks stream at once.
//
// A block has 8 waves (wr, kh): wave (wr, kh) owns W rows [64*tile + 16*wr, +16) and, of every
// chunk of 256 columns, the half kh.  W goes from global memory straight into MFMA operands (a W
// element is used by one wave only), three chunks ahead of its use; the x chunk [rows, 256] is
// staged in LDS once per block, double-buffered, and read from there by all waves.  The two
// column halves are added through LDS in a fixed order; with ksplit > 1 the output is
// [ksplit][M][N] float, partial products that the reader adds in that order.
//
// v_mfma_f32_16x16x32_bf16 with A = 16 rows of W, B = 16 rows of x: the accumulator of row tile
// mt holds y^T[n = lc*4+e][m = mt*16 + li].
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define T64_KC 256                  // columns of a chunk
#define T64_XS (T64_KC + 16)        // LDS row length: 16-byte reads of 16 rows fall on different banks
#define T64_AHEAD 3                 // chunks of W in flight beyond the one in use

template <int MT, typename OutT, bool PAIRS>
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))   // one block a compute unit, 256 registers a lane
gemm_tile64_kernel(OutT* __restrict__ y, const bf16_t* __restrict__ x, const bf16_t* __restrict__ W,
                   int M, int N, int K, long long ldx, long long ldy, int k_per, int act) {
  constexpr int ROWS = MT * 16;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16_t (*xs)[ROWS * T64_XS] = (bf16_t (*)[ROWS * T64_XS])smem;   // [2][ROWS][T64_XS]
  const int tid = threadIdx.x;
  const int wave = tid >> 6, lane = tid & 63, li = lane & 15, lc = lane >> 4;
  const int wr = wave & 3, kh = wave >> 2;
  const int k_begin = blockIdx.y * k_per, k_end = min(K, k_begin + k_per);
  const int n_chunks = (k_end - k_begin + T64_KC - 1) / T64_KC;
  y += (long long)blockIdx.y * M * ldy;
  const bf16x8 zero = {0, 0, 0, 0, 0, 0, 0, 0};

  // Every load of the main loop is unconditional (addresses are clamped instead): a load inside a
  // branch makes the compiler wait for all loads in flight at the join, which would empty the
  // queue of W every round.  Rows of W beyond N and rows of x beyond M read a valid row and feed
  // outputs that are never stored; columns beyond the block's share are zero in x (W there is
  // some other finite weight, times zero); chunks beyond the last read the last one again.
  const int n = blockIdx.x * 64 + wr * 16 + li;
  const bf16_t* wrow = W + (long long)(n < N ? n : 0) * K;
  const int wk0 = kh * 128 + lc * 8;
  auto load_w = [&](int chunk, bf16x8 (&a)[4]) {
    const int k = k_begin + min(chunk, n_chunks - 1) * T64_KC + wk0;
#pragma unroll
    for (int i = 0; i < 4; ++i) a[i] = *(const bf16x8*)(wrow + min(k + i * 32, K - 8));
  };
  // x: thread t stages pieces t, t + 512, ...: piece p is row p / 32, columns (p % 32) * 8 .. + 7
  const int x_row = tid >> 5, x_col = (tid & 31) * 8;
  auto load_x = [&](int chunk, bf16x8 (&v)[MT]) {
    const int k = min(k_begin + min(chunk, n_chunks - 1) * T64_KC + x_col, K - 8);
#pragma unroll
    for (int j = 0; j < MT; ++j) v[j] = *(const bf16x8*)(x + (long long)min(x_row + 16 * j, M - 1) * ldx + k);
  };
  auto store_x = [&](int chunk, const bf16x8 (&v)[MT]) {
    const bool inside = k_begin + chunk * T64_KC + x_col < k_end;
#pragma unroll
    for (int j = 0; j < MT; ++j)
      *(bf16x8*)(&xs[chunk & 1][(x_row + 16 * j) * T64_XS + x_col]) = inside ? v[j] : zero;
  };

  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto multiply = [&](int buf, const bf16x8 (&a)[4]) {
    const bf16_t* xb = &xs[buf][li * T64_XS + wk0];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const bf16x8 b = *(const bf16x8*)(xb + mt * 16 * T64_XS + i * 32);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[i], b, acc[mt], 0, 0, 0);
      }
  };

  bf16x8 a0[4], a1[4], a2[4], a3[4], x0[MT], x1[MT];
  load_x(0, x0);
  load_x(1, x1);
  load_w(0, a0);
  load_w(1, a1);
  load_w(2, a2);
  store_x(0, x0);
  load_x(2, x0);
  __syncthreads();
  // one round of the ring: chunk c is in `cur`, c + 3 goes to `far`; the x of chunk c + 1 is in
  // `xn` (asked for two rounds ago) and goes to LDS first, then the x of chunk c + 3 is asked for
  // into the same registers.  Loads come back in the order they were asked for, so nothing here
  // waits for anything younger than two rounds.
  auto round = [&](int c, bf16x8 (&cur)[4], bf16x8 (&far)[4], bf16x8 (&xn)[MT]) {
    __builtin_amdgcn_sched_barrier(0);
    store_x(c + 1, xn);          // beyond the last chunk: zeros into the buffer nobody reads
    __builtin_amdgcn_sched_barrier(0);
    load_x(c + 3, xn);
    load_w(c + T64_AHEAD, far);
    __builtin_amdgcn_sched_barrier(0);   // the loads are asked for before the products, not after
    multiply(c & 1, cur);
    __syncthreads();
  };
  // Four rounds without a way out between them: with an exit after each round the compiler moves
  // the far loads behind the exits, next to their use, and the queue of W runs empty.  Rounds
  // beyond the last chunk multiply zeros.
  for (int c = 0; c < n_chunks; c += 4) {
    round(c, a0, a3, x1);
    round(c + 1, a1, a0, x0);
    round(c + 2, a2, a1, x1);
    round(c + 3, a3, a2, x0);
  }

  // add the two column halves in fixed order (half 0 + half 1) and store
  float* red = (float*)smem;                       // [4 row waves][MT][256]; every wave has left the loop
  if (kh == 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(f32x4*)(red + ((wr * MT + mt) * 256 + lane * 4)) = acc[mt];
  }
  __syncthreads();
  if (kh == 0) {
    const int nb = blockIdx.x * 64 + wr * 16 + lc * 4;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const f32x4 t = *(const f32x4*)(red + ((wr * MT + mt) * 256 + lane * 4));
      f32x4 s = acc[mt];
      s[0] += t[0]; s[1] += t[1]; s[2] += t[2]; s[3] += t[3];
      const int m = mt * 16 + li;
      if (m >= M) continue;
      if (PAIRS) {
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

template <int MT, typename OutT, bool PAIRS>
static int launch_tile64(void* y, const void* x, const void* W, int M, int N, int K, long long ldx, long long ldy,
                         int ksplit, int act, hipStream_t stream) {
  // columns per group: a whole number of chunks, every group with at least one column
  const int chunks = (K + T64_KC - 1) / T64_KC;
  const int k_per = ((chunks + ksplit - 1) / ksplit) * T64_KC;
  if ((long long)k_per * (ksplit - 1) >= K) return (int)hipErrorInvalidValue;
  const size_t shmem = (size_t)2 * MT * 16 * T64_XS * sizeof(bf16_t);   // more than the 4 * MT KB of the final sum
  if (shmem > 64 * 1024) {
    static bool raised = false;  // per instantiation
    if (!raised) {
      hipError_t e = hipFuncSetAttribute((const void*)gemm_tile64_kernel<MT, OutT, PAIRS>,
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
      if (e != hipSuccess) return (int)e;
      raised = true;
    }
  }
  hipLaunchKernelGGL((gemm_tile64_kernel<MT, OutT, PAIRS>), dim3((N + 63) / 64, ksplit), dim3(512), shmem, stream,
                     (OutT*)y, (const bf16_t*)x, (const bf16_t*)W, M, N, K, ldx, ldy, k_per, act);
  return JV_LAUNCH_CHECK();
}

template <typename OutT, bool PAIRS>
static int dispatch_tile64(void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                           long long ldy, int ksplit, int act, hipStream_t s) {
  switch ((M + 15) / 16) {
    case 1: return launch_tile64<1, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, ksplit, act, s);
    case 2: return launch_tile64<2, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, ksplit, act, s);
    case 3: return launch_tile64<3, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, ksplit, act, s);
    case 4: return launch_tile64<4, OutT, PAIRS>(y, x, W, M, N, K, ldx, ldy, ksplit, act, s);
  }
  return (int)hipErrorInvalidValue;
}

// out_f32: 0 -> y is bf16, 1 -> y is float.  x is [M, K] with row stride ldx, M <= 64.
// gate_act: JV_ACT_* (not 0) -> the rows of W alternate gate and up rows and y[m, j] =
//      act(x.W[2j]) * (x.W[2j+1]) is bf16 [M, N/2].
// ksplit > 1 (float output, no activation): K is shared out to ksplit blocks per tile of 64 rows of W
// and y is [ksplit][M][ldy], partial products that the reader adds in that order; refused when
// a group would be left without columns.
extern "C" int jv_gemm_tile64_bf16(void* y, const void* x, const void* W, int M, int N, int K, long long ldx,
                                   long long ldy, int out_f32, int gate_act, int ksplit, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 != 0 || ldx % 8 != 0) return (int)hipErrorInvalidValue;
  if (gate_act && (!jv_act_known(gate_act) || out_f32 || N % 2 != 0 || ksplit != 1)) return (int)hipErrorInvalidValue;
  if (ksplit < 1 || ksplit > 65535 || (ksplit > 1 && !out_f32)) return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  if (gate_act) return dispatch_tile64<bf16_t, true>(y, x, W, M, N, K, ldx, ldy, ksplit, gate_act, s);
  return out_f32 ? dispatch_tile64<float, false>(y, x, W, M, N, K, ldx, ldy, ksplit, 0, s)
                 : dispatch_tile64<bf16_t, false>(y, x, W, M, N, K, ldx, ldy, ksplit, 0, s);
}
