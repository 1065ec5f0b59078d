// Next-token choice on the device: argmax (pyre/scheduler.py:80,94) and
// temperature sampling by the inverse of the cumulative distribution, all in fp32.
// One block per row of logits. A row's result depends on that row alone.
#include <mutex>

#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

// Scratch of pyre_argmax_static: the slices' best values (64 floats per row) followed by
// their indices (64 ints per row) for up to PYRE_ARGMAX_STATIC_MAX_ROWS rows, 128 KB on
// every GPU the library runs on, held until the process ends. In host code this name is a
// stand-in for the symbol, not a device address: the address of a device's copy comes from
// hipGetSymbolAddress (static_scratch_of below) and only that pointer is handed to kernels.
static __device__ __align__(256) unsigned char scratch[PYRE_ARGMAX_STATIC_MAX_ROWS * 128 * 4];

namespace {

constexpr int kThreads = 1024;

// Largest value; among equal values the lowest index (torch.argmax's choice).
// Two stages so that a few rows still fill the chip: kSlices blocks per row each
// reduce a slice of the vocabulary, then one block per row reduces the slices.
constexpr int kSlices = 64;
constexpr int kArgThreads = 256;

__device__ inline void better(float& bv, int& bi, float ov, int oi) {
  if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
}

__device__ inline void block_argmax(float& bv, int& bi, float* sv, int* si) {
  for (int o = kWave / 2; o > 0; o >>= 1) better(bv, bi, __shfl_xor(bv, o, kWave), __shfl_xor(bi, o, kWave));
  const int w = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) { sv[w] = bv; si[w] = bi; }
  __syncthreads();
  if (threadIdx.x == 0)
    for (int i = 1; i < kArgThreads / kWave; ++i) better(bv, bi, sv[i], si[i]);
}

__global__ __launch_bounds__(kArgThreads) void argmax_slices_kernel(const float* __restrict__ logits,
                                                                    size_t row_stride, float* __restrict__ pv,
                                                                    int* __restrict__ pi, int vocab) {
  __shared__ float sv[kArgThreads / kWave];
  __shared__ int si[kArgThreads / kWave];
  const float* row = logits + blockIdx.x * row_stride;
  const int per = (vocab + kSlices - 1) / kSlices;
  const int begin = min(vocab, static_cast<int>(blockIdx.y) * per), end = min(vocab, begin + per);
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = begin + threadIdx.x; i < end; i += kArgThreads) {
    const float v = row[i];
    if (bi == 0x7fffffff) { bv = v; bi = i; } else better(bv, bi, v, i);
  }
  block_argmax(bv, bi, sv, si);
  if (threadIdx.x == 0) {
    pv[blockIdx.x * kSlices + blockIdx.y] = bv;
    pi[blockIdx.x * kSlices + blockIdx.y] = bi;
  }
}

__global__ __launch_bounds__(kWave) void argmax_final_kernel(const float* __restrict__ pv,
                                                             const int* __restrict__ pi, int* __restrict__ out) {
  float bv = pv[blockIdx.x * kSlices + threadIdx.x];
  int bi = pi[blockIdx.x * kSlices + threadIdx.x];
  for (int o = kWave / 2; o > 0; o >>= 1) better(bv, bi, __shfl_xor(bv, o, kWave), __shfl_xor(bi, o, kWave));
  if (threadIdx.x == 0) out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
}

// p_i = exp((x_i - max) / T) / sum;  token = first i with cumsum(p)_i > u, u in [0, 1).
// Thread t owns the contiguous slice [t * per, (t + 1) * per) of the vocabulary, so that the
// cumulative sum runs in vocabulary order: the sum before slice t is (sum of the slices of the
// waves before t's, added wave by wave) + (sum of the slices before t in its wave), which never
// decreases with t. A thread whose slice may hold the target walks it element by element from
// that sum; the lowest token at which a walk passes the target is the result. If rounding lets
// every walk end at or below the target, the result is the last token of non-zero probability
// of the last slice that was walked.
__global__ __launch_bounds__(kThreads) void sample_kernel(const float* __restrict__ logits,
                                                          size_t row_stride,
                                                          const float* __restrict__ temperature,
                                                          const float* __restrict__ uniform,
                                                          int* __restrict__ out, int vocab) {
  constexpr int kWaves = kThreads / kWave;
  __shared__ float scratch[16];
  __shared__ float slice_sum[kThreads];
  __shared__ float slice_before[kThreads];  // sum of the slices before this one in its wave
  __shared__ float wave_before[kWaves + 1]; // sum of the waves before this one; [kWaves]: the total
  __shared__ int passed, missed;
  const int r = blockIdx.x, tid = threadIdx.x, w = tid / kWave;
  if (!(temperature[r] > 0.f)) return;  // greedy rows keep the argmax already in out[r]
  const float* row = logits + r * row_stride;
  const float inv_t = 1.f / temperature[r];
  const int per = (vocab + kThreads - 1) / kThreads;
  const int begin = min(vocab, tid * per), end = min(vocab, begin + per);

  float mx = -INFINITY;
  for (int i = begin; i < end; ++i) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, scratch);

  float s = 0.f;
  for (int i = begin; i < end; ++i) s += expf((row[i] - mx) * inv_t);
  slice_sum[tid] = s;
  if (tid == 0) { passed = 0x7fffffff; missed = -1; }
  __syncthreads();
  if ((tid & (kWave - 1)) == 0) {
    float run = 0.f;
    for (int j = 0; j < kWave; ++j) { slice_before[tid + j] = run; run += slice_sum[tid + j]; }
    scratch[w] = run;
  }
  __syncthreads();
  if (tid == 0) {
    float run = 0.f;
    for (int j = 0; j < kWaves; ++j) { wave_before[j] = run; run += scratch[j]; }
    wave_before[kWaves] = run;
  }
  __syncthreads();
  const float target = uniform[r] * wave_before[kWaves];
  const float before = wave_before[w] + slice_before[tid];
  // The slice that holds the target starts at or below it and ends above it; the ends are
  // taken a little generously, since a walk's sum and the slice's own differ by rounding.
  if (s > 0.f && before <= target && (before + s) >= target * (1.f - 1e-5f)) {
    float run = before;
    int pick = -1, last = -1;
    for (int i = begin; i < end; ++i) {
      const float p = expf((row[i] - mx) * inv_t);
      run += p;
      if (p > 0.f) {
        last = i;
        if (run > target) { pick = i; break; }
      }
    }
    if (pick >= 0) atomicMin(&passed, pick);
    else atomicMax(&missed, last);
  }
  __syncthreads();
  if (tid == 0) {
    int pick = passed != 0x7fffffff ? passed : missed;
    if (pick < 0) {  // nobody walked: the last token that can be drawn at all
      for (int i = vocab - 1; i >= 0 && pick < 0; --i)
        if (expf((row[i] - mx) * inv_t) > 0.f) pick = i;
    }
    out[r] = pick < 0 ? 0 : pick;
  }
}

// tokens[i] = ids[src[i]] for the rows whose token is a result still on the device.
__global__ __launch_bounds__(256) void feed_tokens_kernel(int* __restrict__ tokens, const int* __restrict__ src,
                                                           const int* __restrict__ ids, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n && src[i] >= 0) tokens[i] = ids[src[i]];
}

}  // namespace

extern "C" int pyre_feed_tokens(int* tokens, const int* src, const int* ids, int n, hipStream_t stream) {
  if (n <= 0) return 0;
  hipLaunchKernelGGL(feed_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, tokens, src, ids, n);
  return check_launch("feed_tokens");
}

// scratch: m * 64 floats followed by m * 64 ints.
extern "C" int pyre_argmax(const float* logits, long row_stride, int* out, void* scratch, int m, int vocab,
                           hipStream_t stream) {
  PYRE_REQUIRE(vocab > 0 && row_stride >= vocab, "argmax: bad sizes");
  PYRE_REQUIRE(m <= 65535, "argmax: too many rows");
  if (m <= 0) return 0;
  static_assert(kSlices == kWave, "the final stage reduces one slice per lane");
  float* pv = static_cast<float*>(scratch);
  int* pi = reinterpret_cast<int*>(pv + static_cast<size_t>(m) * kSlices);
  hipLaunchKernelGGL(argmax_slices_kernel, dim3(m, kSlices), dim3(kArgThreads), 0, stream, logits,
                     static_cast<size_t>(row_stride), pv, pi, vocab);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(m), dim3(kWave), 0, stream, pv, pi, out);
  return check_launch("argmax");
}

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_static_mutex;
void* g_static_scratch[kMaxDevices] = {};  // the address of `scratch` on each device, once asked for

// The current device's copy of `scratch`. Every GPU holds its own copy of the array at its own
// address, so the address is asked for once per device, with that device current.
int static_scratch_of(int device, void** ptr) {
  std::lock_guard<std::mutex> guard(g_static_mutex);
  if (!g_static_scratch[device]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    PYRE_REQUIRE(e == hipSuccess && p, "argmax_static: hipGetSymbolAddress on device %d: %s", device,
                 hipGetErrorString(e));
    g_static_scratch[device] = p;
  }
  *ptr = g_static_scratch[device];
  return 0;
}

// The current device's copy of `scratch`, looked up at the first call on that device.
int static_scratch_here(void** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  PYRE_REQUIRE(e == hipSuccess, "argmax_static: hipGetDevice: %s", hipGetErrorString(e));
  PYRE_REQUIRE(device >= 0 && device < kMaxDevices, "argmax_static: device %d is beyond the %d this entry point knows",
               device, kMaxDevices);
  return static_scratch_of(device, ptr);
}

}  // namespace

extern "C" int pyre_argmax_static_init() {
  void* base = nullptr;
  return static_scratch_here(&base);
}

extern "C" int pyre_argmax_static(const float* logits, long row_stride, int* out, int m, int vocab,
                                  hipStream_t stream) {
  PYRE_REQUIRE(vocab > 0 && row_stride >= vocab, "argmax_static: bad sizes");
  PYRE_REQUIRE(m <= PYRE_ARGMAX_STATIC_MAX_ROWS,
               "argmax_static: %d rows; the built-in scratch holds %d (use pyre_argmax with scratch of your own)", m,
               PYRE_ARGMAX_STATIC_MAX_ROWS);
  if (m <= 0) return 0;
  void* base = nullptr;
  if (int rc = static_scratch_here(&base)) return rc;
  // Nothing has to start at zero: the first stage writes all 64 slices of every row before
  // the second stage reads them, whatever an earlier (larger) call left behind.
  float* pv = static_cast<float*>(base);
  int* pi = reinterpret_cast<int*>(pv + static_cast<size_t>(m) * kSlices);
  hipLaunchKernelGGL(argmax_slices_kernel, dim3(m, kSlices), dim3(kArgThreads), 0, stream, logits,
                     static_cast<size_t>(row_stride), pv, pi, vocab);
  hipLaunchKernelGGL(argmax_final_kernel, dim3(m), dim3(kWave), 0, stream, pv, pi, out);
  return check_launch("argmax_static");
}

extern "C" int pyre_sample(const float* logits, long row_stride, const float* temperature,
                           const float* uniform, int* out, int m, int vocab, hipStream_t stream) {
  PYRE_REQUIRE(vocab > 0 && row_stride >= vocab, "sample: bad sizes");
  if (m <= 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(m), dim3(kThreads), 0, stream, logits,
                     static_cast<size_t>(row_stride), temperature, uniform, out, vocab);
  return check_launch("sample");
}
