// Token choice from float logits [M, V] in two stages: many blocks per row each find the winner
// of a slice of the vocabulary, then one small block per row picks among them.
//   temperature[r] <= 0 : greedy, the lowest index among the maxima;
//   temperature[r] >  0 : a draw from softmax(logits / temperature) by the Gumbel-max
//     rule: argmax_i( logits[i] / T + g_i ), g_i = -log(-log(u_i)), where u_i in (0,1)
//     comes from a counter-based generator keyed by (key[r], i).  The draw depends on
//     the row's key and logits only, not on the batch it is in.
#include "common.h"
#include "sampling.h"

#include <mutex>
#include <stdio.h>

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float uniform_open01(uint64_t key, uint32_t i) {
  const uint64_t bits = mix64(mix64(key) ^ (uint64_t)i * 0xD1342543DE82EF95ull);
  // 24 high bits -> (0, 1): never 0, never 1
  return ((float)(bits >> 40) + 0.5f) * (1.0f / 16777216.0f);
}

struct Best { float v; int i; };
__device__ __forceinline__ bool better(float v, int i, float bv, int bi) { return v > bv || (v == bv && i < bi); }

// Reduces (value, index) over the block; thread 0 returns the winner.
__device__ __forceinline__ Best block_best(float best, int best_i) {
  __shared__ float bv[4];
  __shared__ int bi[4];
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (better(ov, oi, best, best_i)) { best = ov; best_i = oi; }
  }
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  if (lane == 0) { bv[wid] = best; bi[wid] = best_i; }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int w = 1; w < (int)(blockDim.x >> 6); ++w)
      if (better(bv[w], bi[w], best, best_i)) { best = bv[w]; best_i = bi[w]; }
  return Best{best, best_i};
}

// Stage 1: grid (chunks, rows); block (c, r) scans columns [c * chunk, (c+1) * chunk) of row r and
// writes its winner to part[r, c].  Stage 2: grid (rows); reduces the chunks' winners.
__global__ void __launch_bounds__(256)
sample_stage1_kernel(float* __restrict__ part_v, int* __restrict__ part_i, const float* __restrict__ logits,
                     long long row_stride, int V, int chunk, const float* __restrict__ temperature,
                     const unsigned long long* __restrict__ keys) {
  const long long r = blockIdx.y;
  const int c = blockIdx.x;
  const float* row = logits + r * row_stride;
  const float temp = temperature ? temperature[r] : 0.f;
  const uint64_t key = keys ? keys[r] : 0ull;
  const float inv_t = temp > 0.f ? 1.f / temp : 1.f;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  const int end = (c + 1) * chunk < V ? (c + 1) * chunk : V;
  for (int i = c * chunk + threadIdx.x; i < end; i += blockDim.x) {
    float v = row[i] * inv_t;
    if (temp > 0.f) v += -logf(-logf(uniform_open01(key, (uint32_t)i)));
    if (better(v, i, best, best_i)) { best = v; best_i = i; }
  }
  const Best b = block_best(best, best_i);
  if (threadIdx.x == 0) {
    part_v[r * gridDim.x + c] = b.v;
    part_i[r * gridDim.x + c] = b.i;
  }
}

__global__ void __launch_bounds__(64)
sample_stage2_kernel(int* __restrict__ out, const float* __restrict__ part_v, const int* __restrict__ part_i,
                     int chunks, int V) {
  const long long r = blockIdx.x;
  float best = -INFINITY;
  int best_i = 0x7fffffff;
  for (int c = threadIdx.x; c < chunks; c += 64) {
    const float v = part_v[r * chunks + c];
    const int i = part_i[r * chunks + c];
    if (better(v, i, best, best_i)) { best = v; best_i = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, 64);
    const int oi = __shfl_xor(best_i, o, 64);
    if (better(ov, oi, best, best_i)) { best = ov; best_i = oi; }
  }
  // NaN logits never win a comparison; a row of them is reported as V
  if (threadIdx.x == 0) out[r] = best_i < V ? best_i : V;
}

#define SAMPLE_MAX_CHUNKS 64

static int sample_launch(int* out, const float* logits, long long row_stride, int n_rows, int V,
                         const float* temperature, const unsigned long long* keys, void* scratch,
                         hipStream_t stream) {
  int chunks = (V + 4095) / 4096;  // at least 4096 columns per block
  if (chunks > SAMPLE_MAX_CHUNKS) chunks = SAMPLE_MAX_CHUNKS;
  const int chunk = (V + chunks - 1) / chunks;
  float* pv = (float*)scratch;
  int* pi = (int*)(pv + (long long)n_rows * SAMPLE_MAX_CHUNKS);
  hipLaunchKernelGGL(sample_stage1_kernel, dim3(chunks, n_rows), dim3(256), 0, stream, pv, pi, logits, row_stride,
                     V, chunk, temperature, keys);
  int e = JV_LAUNCH_CHECK();
  if (e) return e;
  hipLaunchKernelGGL(sample_stage2_kernel, dim3(n_rows), dim3(64), 0, stream, out, pv, pi, chunks, V);
  return JV_LAUNCH_CHECK();
}

// scratch: SAMPLE_MAX_CHUNKS * n_rows floats followed by as many ints (jv_sample_scratch_bytes)
extern "C" long long jv_sample_scratch_bytes(int n_rows) { return (long long)n_rows * SAMPLE_MAX_CHUNKS * 8; }

extern "C" int jv_sample(int* out, const float* logits, long long row_stride, int n_rows, int V,
                         const float* temperature, const unsigned long long* keys, void* scratch,
                         void* stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || !scratch || n_rows > 65535) return (int)hipErrorInvalidValue;
  return sample_launch(out, logits, row_stride, n_rows, V, temperature, keys, scratch, (hipStream_t)stream);
}

// ---------------------------------------------------------------------------------------------
// The same choice of tokens without a workspace from the caller: the stage-one winners go to a
// fixed array in device memory that the library itself holds, on every GPU it runs on, until the
// process ends (JV_SAMPLE_NOALLOC_MAX_ROWS * 64 chunks * 8 bytes = 512 KiB).  Nothing is allocated
// or freed here or by anything this calls.  Stage one writes every (row, chunk) entry that stage
// two reads, so nothing has to start at zero and what an earlier call left does not matter.  All
// calls on one GPU share the array: two calls that overlap there (different streams, or graphs
// replayed at the same time) race on it.
static __device__ __align__(256) unsigned char sample_noalloc_scratch[JV_SAMPLE_NOALLOC_MAX_ROWS * SAMPLE_MAX_CHUNKS * 8];

#define SAMPLE_NOALLOC_MAX_DEVICES 64
// The array's address on each device.  In host code the array's name is only a stand-in for the
// symbol; the address a kernel can use comes from hipGetSymbolAddress, and each GPU has its own.
static void* sample_noalloc_ptr[SAMPLE_NOALLOC_MAX_DEVICES];
static std::mutex sample_noalloc_mutex;
static thread_local char sample_noalloc_error[256];

extern "C" const char* jv_sample_noalloc_last_error(void) { return sample_noalloc_error; }

// Resolves the array's address on the current device (once per device).  Returns 0 or a hipError_t.
static int sample_noalloc_resolve(void** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) {
    snprintf(sample_noalloc_error, sizeof sample_noalloc_error, "jv_sample_noalloc: hipGetDevice failed: %s",
             hipGetErrorString(e));
    return (int)e;
  }
  if (dev < 0 || dev >= SAMPLE_NOALLOC_MAX_DEVICES) {
    snprintf(sample_noalloc_error, sizeof sample_noalloc_error,
             "jv_sample_noalloc: device %d is beyond the %d devices this entry point keeps an address for", dev,
             SAMPLE_NOALLOC_MAX_DEVICES);
    return (int)hipErrorInvalidDevice;
  }
  std::lock_guard<std::mutex> lock(sample_noalloc_mutex);
  if (!sample_noalloc_ptr[dev]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(sample_noalloc_scratch));
    if (e != hipSuccess || !p) {
      snprintf(sample_noalloc_error, sizeof sample_noalloc_error,
               "jv_sample_noalloc: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return e != hipSuccess ? (int)e : (int)hipErrorInvalidSymbol;
    }
    sample_noalloc_ptr[dev] = p;
  }
  *ptr = sample_noalloc_ptr[dev];
  return 0;
}

extern "C" int jv_sample_noalloc_init(void) {
  void* p = nullptr;
  sample_noalloc_error[0] = 0;
  return sample_noalloc_resolve(&p);
}

extern "C" int jv_sample_noalloc(int* out, const float* logits, long long row_stride, int n_rows, int V,
                                 const float* temperature, const unsigned long long* keys, void* stream) {
  sample_noalloc_error[0] = 0;
  if (n_rows <= 0) return 0;
  if (n_rows > JV_SAMPLE_NOALLOC_MAX_ROWS) {
    snprintf(sample_noalloc_error, sizeof sample_noalloc_error,
             "jv_sample_noalloc: %d rows exceed the maximum of %d that the fixed %d KiB array holds; "
             "call it on slices of the rows or use jv_sample with a workspace", n_rows, JV_SAMPLE_NOALLOC_MAX_ROWS,
             JV_SAMPLE_NOALLOC_MAX_ROWS * SAMPLE_MAX_CHUNKS * 8 / 1024);
    return (int)hipErrorInvalidValue;
  }
  if (V <= 0 || !out || !logits || (temperature && !keys)) {
    snprintf(sample_noalloc_error, sizeof sample_noalloc_error,
             "jv_sample_noalloc: needs out, logits, a vocabulary of at least 1 and keys wherever temperatures are given");
    return (int)hipErrorInvalidValue;
  }
  void* scratch = nullptr;
  const int e = sample_noalloc_resolve(&scratch);
  if (e) return e;
  // from here on only the resolved address is used, never the array's name
  return sample_launch(out, logits, row_stride, n_rows, V, temperature, keys, scratch, (hipStream_t)stream);
}
