// Next-token choice on the device: argmax (pyre/scheduler.py:80,94) and
// temperature sampling by the inverse of the cumulative distribution, all in fp32.
// One block per row of logits. A row's result depends on that row alone.
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

constexpr int kThreads = 1024;

// Largest value; among equal values the lowest index (torch.argmax's choice).
__global__ __launch_bounds__(kThreads) void argmax_kernel(const float* __restrict__ logits,
                                                          size_t row_stride, int* __restrict__ out,
                                                          int vocab) {
  __shared__ float best_v[kThreads / kWave];
  __shared__ int best_i[kThreads / kWave];
  const float* row = logits + blockIdx.x * row_stride;
  float bv = -INFINITY;
  int bi = 0x7fffffff;
  for (int i = threadIdx.x; i < vocab; i += kThreads) {
    const float v = row[i];
    if (v > bv || (v == bv && i < bi) || bi == 0x7fffffff) { bv = v; bi = i; }
  }
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const float ov = __shfl_xor(bv, o, kWave);
    const int oi = __shfl_xor(bi, o, kWave);
    if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
  }
  const int w = threadIdx.x / kWave;
  if ((threadIdx.x & (kWave - 1)) == 0) { best_v[w] = bv; best_i[w] = bi; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < kThreads / kWave; ++i)
      if (best_v[i] > bv || (best_v[i] == bv && best_i[i] < bi)) { bv = best_v[i]; bi = best_i[i]; }
    out[blockIdx.x] = bi == 0x7fffffff ? 0 : bi;
  }
}

// p_i = exp((x_i - max) / T) / sum;  token = first i with cumsum(p)_i > u, u in [0, 1).
// Thread t owns the contiguous slice [t * per, (t + 1) * per) of the vocabulary,
// so that the cumulative sum runs in vocabulary order.
__global__ __launch_bounds__(kThreads) void sample_kernel(const float* __restrict__ logits,
                                                          size_t row_stride,
                                                          const float* __restrict__ temperature,
                                                          const float* __restrict__ uniform,
                                                          int* __restrict__ out, int vocab) {
  __shared__ float scratch[16];
  __shared__ float slice_sum[kThreads];
  __shared__ int chosen;
  const int r = blockIdx.x, tid = threadIdx.x;
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
  if (tid == 0) chosen = -1;
  __syncthreads();

  if (tid == 0) {
    float total = 0.f;
    for (int t = 0; t < kThreads; ++t) total += slice_sum[t];
    const float target = uniform[r] * total;
    // Find the slice in which the running sum passes the target, then the element.
    float run = 0.f;
    int t = 0;
    for (; t < kThreads - 1; ++t) {
      if (run + slice_sum[t] > target) break;
      run += slice_sum[t];
    }
    int b = min(vocab, t * per), e = min(vocab, b + per);
    // Rounding may leave the target just beyond the last slice's sum: fall back
    // to the last token with non-zero probability.
    int pick = -1;
    for (int i = b; i < e; ++i) {
      run += expf((row[i] - mx) * inv_t);
      if (run > target) { pick = i; break; }
    }
    if (pick < 0) {
      for (int i = vocab - 1; i >= 0; --i)
        if (expf((row[i] - mx) * inv_t) > 0.f) { pick = i; break; }
    }
    chosen = pick < 0 ? 0 : pick;
    out[r] = chosen;
  }
}

}  // namespace

extern "C" int pyre_argmax(const float* logits, long row_stride, int* out, int m, int vocab,
                           hipStream_t stream) {
  PYRE_REQUIRE(vocab > 0 && row_stride >= vocab, "argmax: bad sizes");
  if (m <= 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(m), dim3(kThreads), 0, stream, logits,
                     static_cast<size_t>(row_stride), out, vocab);
  return check_launch("argmax");
}

extern "C" int pyre_sample(const float* logits, long row_stride, const float* temperature,
                           const float* uniform, int* out, int m, int vocab, hipStream_t stream) {
  PYRE_REQUIRE(vocab > 0 && row_stride >= vocab, "sample: bad sizes");
  if (m <= 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(m), dim3(kThreads), 0, stream, logits,
                     static_cast<size_t>(row_stride), temperature, uniform, out, vocab);
  return check_launch("sample");
}
