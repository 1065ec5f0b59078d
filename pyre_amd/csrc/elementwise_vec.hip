// Vectorised forms of the row kernels for the common case (widths that are
// multiples of 4, no pending bias in the norm, full-head rotary): same formulas and
// the same order of additions as elementwise.hip, 16 bytes per load where the
// general kernels load one element. The entry points in elementwise.hip try these
// first and fall back to the general kernels.
#include "pyre_common.h"
#include "pyre_vec.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

// The same loads and stores past the caches, for rows that are read and written once in a step of
// many rows (more bytes than the caches hold).
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef unsigned u32x2_t __attribute__((ext_vector_type(2)));
template <typename T> struct Stream4;
template <> struct Stream4<float> {
  static __device__ inline float4 load(const float* p) {
    const f32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
    return float4{v[0], v[1], v[2], v[3]};
  }
  static __device__ inline void store(float* p, float4 v) {
    __builtin_nontemporal_store(f32x4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<f32x4_t*>(p));
  }
};
template <> struct Stream4<bf16> {
  static __device__ inline float4 load(const bf16* p) {
    const u32x2_t u = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
    return float4{__uint_as_float(u[0] << 16), __uint_as_float(u[0] & 0xffff0000u), __uint_as_float(u[1] << 16),
                  __uint_as_float(u[1] & 0xffff0000u)};
  }
  static __device__ inline void store(bf16* p, float4 v) {
    __builtin_nontemporal_store(u32x2_t{pack_bf16x2(v.x, v.y), pack_bf16x2(v.z, v.w)}, reinterpret_cast<u32x2_t*>(p));
  }
};

// ---------------------------------------------------------------------------
// add + RMSNorm, one block per row, the row kept in registers between the passes.
// ---------------------------------------------------------------------------
constexpr int kNormMaxVec = 8;  // float4 per thread

// THREADS = 256 keeps up to 8192 elements of a row in registers and suits many rows;
// THREADS = 1024 gives a short row one float4 per thread, so that all loads of a
// decode step's few rows are in flight at once.
//
// The sum of squares is added up in an order that the row's width alone fixes, whichever
// variant runs: a row wider than 1024 elements is summed as 1024 threads would (thread t
// adds its pieces t, t + 1024, ... in ascending order; every 64 consecutive threads are
// reduced by the butterfly of wave_sum; the 16 results are added in ascending order).
// The 256-thread variant then plays VIRT = 4 of those threads per thread: t = thread +
// 256 j. A position's result therefore does not depend on how many rows share the step.
template <typename TD, typename TG, typename TO, int THREADS, int VIRT, bool STREAM>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_vec_kernel(
    float* __restrict__ resid, const TD* __restrict__ delta, int n_partials, size_t partial_stride,
    const TG* __restrict__ gain, TO* __restrict__ out, const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x, r_in = rows ? rows[r_out] : r_out;
  const size_t in_off = static_cast<size_t>(r_in) * hidden;
  const int nvec = hidden / 4;
  float4 v[kNormMaxVec];
  float ss[VIRT];
#pragma unroll
  for (int j = 0; j < VIRT; ++j) ss[j] = 0.f;
#pragma unroll
  for (int i = 0; i < kNormMaxVec; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) break;
    float4 x = STREAM ? Stream4<float>::load(resid + in_off + 4 * c) : Vec4<float>::load(resid + in_off + 4 * c);
    if (delta) {
      float4 d;
      if (STREAM) {  // the same sums in the same order
        d = Stream4<TD>::load(delta + in_off + 4 * c);
        for (int p = 1; p < n_partials; ++p) d = add4(d, Stream4<TD>::load(delta + p * partial_stride + in_off + 4 * c));
      } else {
        d = sum_partials4<TD>(delta + in_off + 4 * c, partial_stride, n_partials);
      }
      x = add4(x, d);
      if (!rows) {
        if (STREAM) Stream4<float>::store(resid + in_off + 4 * c, x);
        else Vec4<float>::store(resid + in_off + 4 * c, x);
      }
    }
    v[i] = x;
    // explicit fused multiply-adds: the same roundings in every variant of the kernel
    ss[i % VIRT] = fmaf(x.w, x.w, fmaf(x.z, x.z, fmaf(x.y, x.y, fmaf(x.x, x.x, ss[i % VIRT]))));
  }
  float total;
  if (VIRT == 1) {
    total = block_sum(ss[0], scratch);
  } else {
    // the waves of the threads this thread stands for are wave + (THREADS / 64) j
    const int w = threadIdx.x / kWave;
#pragma unroll
    for (int j = 0; j < VIRT; ++j) {
      const float s = wave_sum(ss[j]);
      if ((threadIdx.x & (kWave - 1)) == 0) scratch[w + (THREADS / kWave) * j] = s;
    }
    __syncthreads();
    total = 0.f;
    for (int i = 0; i < VIRT * THREADS / kWave; ++i) total += scratch[i];
  }
  const float inv = rsqrtf(total / static_cast<float>(hidden) + eps);
  const size_t out_off = static_cast<size_t>(r_out) * hidden;
#pragma unroll
  for (int i = 0; i < kNormMaxVec; ++i) {
    const int c = threadIdx.x + i * THREADS;
    if (c >= nvec) break;
    const float4 gn = Vec4<TG>::load(gain + 4 * c);
    const float4 x = v[i];
    const float4 y{x.x * inv * gn.x, x.y * inv * gn.y, x.z * inv * gn.z, x.w * inv * gn.w};
    if (STREAM) Stream4<TO>::store(out + out_off + 4 * c, y);
    else Vec4<TO>::store(out + out_off + 4 * c, y);
  }
}

// ---------------------------------------------------------------------------
// rotary + cache write, four pairs per item; grid (tokens, ceil(items / 256)).
// ---------------------------------------------------------------------------
template <typename TI, typename TC, bool STREAM>
__global__ __launch_bounds__(256) void rope_kv_write_vec_kernel(
    const TI* __restrict__ qkv, int n_partials, size_t partial_stride, const void* __restrict__ bias,
    int bias_dt, TC* __restrict__ q_out, TC* __restrict__ k_cache, TC* __restrict__ v_cache,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, const int* __restrict__ positions,
    const int* __restrict__ slots, int nq, int nkv, int hd, int page_size, int write_kv) {
  const int n = blockIdx.x;
  const int half = hd / 2, hv = half / 4;            // vec4 pairs per head
  const int n_rot = (nq + nkv) * hv, n_items = n_rot + nkv * (hd / 4);
  const int it = blockIdx.y * 256 + threadIdx.x;
  if (it >= n_items) return;
  const int width = (nq + 2 * nkv) * hd;
  const size_t in_row = static_cast<size_t>(n) * width;
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;

  auto value4 = [&](int col) {
    float4 v;
    if (STREAM) {  // the product's rows of a step of many tokens are read once: past the caches
      v = Stream4<TI>::load(qkv + in_row + col);
      for (int p = 1; p < n_partials; ++p) v = add4(v, Stream4<TI>::load(qkv + p * partial_stride + in_row + col));
    } else {
      v = sum_partials4<TI>(qkv + in_row + col, partial_stride, n_partials);
    }
    if (bias) {  // col is a multiple of 4: one load of four
      v = add4(v, bias_dt == kF32 ? Vec4<float>::load(static_cast<const float*>(bias) + col)
                                  : Vec4<bf16>::load(static_cast<const bf16*>(bias) + col));
    }
    return v;
  };

  if (it < n_rot) {
    const int head = it / hv, j = 4 * (it % hv);
    if (head >= nq && slot < 0) return;
    const int base = head * hd;
    const float4 x1 = value4(base + j), x2 = value4(base + j + half);
    const size_t t = static_cast<size_t>(positions[n]) * half + j;
    const float4 c = Vec4<float>::load(cos_t + t), s = Vec4<float>::load(sin_t + t);
    float4 a, b;
    rotate_pair(x1.x, x2.x, c.x, s.x, a.x, b.x);
    rotate_pair(x1.y, x2.y, c.y, s.y, a.y, b.y);
    rotate_pair(x1.z, x2.z, c.z, s.z, a.z, b.z);
    rotate_pair(x1.w, x2.w, c.w, s.w, a.w, b.w);
    TC* dst = head < nq ? q_out + static_cast<size_t>(n) * nq * hd + base
                        : k_cache + ((static_cast<size_t>(page) * nkv + (head - nq)) * page_size + off) * hd;
    Vec4<TC>::store(dst + j, a);
    Vec4<TC>::store(dst + j + half, b);
  } else if (slot >= 0) {
    const int e = 4 * (it - n_rot);
    const int kvh = e / hd, d = e % hd;
    const float4 v = value4((nq + nkv) * hd + e);
    TC* row = v_cache + ((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size;
    row[off] = from_float<TC>(v.x);
    row[page_size + off] = from_float<TC>(v.y);
    row[2 * static_cast<size_t>(page_size) + off] = from_float<TC>(v.z);
    row[3 * static_cast<size_t>(page_size) + off] = from_float<TC>(v.w);
    // the step's last token of a page leaves nothing of the page's previous owner behind it
    if (ends_its_page_run(slots, n, gridDim.x, slot, page_size)) {
#pragma unroll
      for (int r = 0; r < 4; ++r) zero_tail(row + r * static_cast<size_t>(page_size), off + 1, page_size);
    }
  }
}

// ---------------------------------------------------------------------------
// SiLU-gate, four features per thread; eight, in 16-byte loads that go past the caches,
// for bfloat16 without partial sums (a prompt portion's gate/up product, read once).
// ---------------------------------------------------------------------------
__device__ inline float silu_gate(float g, float u) { return g / (1.f + expf(-g)) * u; }
// For results that are rounded to bfloat16: the hardware's exponential and reciprocal (errors of a
// few units in the last place of float32), as in the epilogue of the decode step's gate/up product.
__device__ inline float silu_gate_fast(float g, float u) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u; }

template <typename TI, typename TO>
__global__ __launch_bounds__(256) void silu_mul_vec_kernel(const TI* __restrict__ gu, int n_partials,
                                                           size_t partial_stride, TO* __restrict__ out,
                                                           size_t total4, int inter) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const int per_row = inter / 4;
  const size_t n = i / per_row, c = 4 * (i % per_row);
  const size_t gi = n * 2 * inter + c, ui = gi + inter;
  float4 g = Vec4<TI>::load(gu + gi), u = Vec4<TI>::load(gu + ui);
  for (int p = 1; p < n_partials; ++p) {
    g = add4(g, Vec4<TI>::load(gu + p * partial_stride + gi));
    u = add4(u, Vec4<TI>::load(gu + p * partial_stride + ui));
  }
  Vec4<TO>::store(out + n * inter + c, float4{silu_gate(g.x, u.x), silu_gate(g.y, u.y), silu_gate(g.z, u.z),
                                              silu_gate(g.w, u.w)});
}

__global__ __launch_bounds__(256) void silu_mul_stream_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out,
                                                              size_t total8, int inter) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total8) return;
  const int per_row = inter / 8;
  const size_t n = i / per_row, c = 8 * (i % per_row);
  const bf16* gp = gu + n * 2 * inter + c;
  const u32x4 g = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gp));
  const u32x4 u = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(gp + inter));
  u32x4 y;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float lo = silu_gate_fast(__uint_as_float(g[j] << 16), __uint_as_float(u[j] << 16));
    const float hi = silu_gate_fast(__uint_as_float(g[j] & 0xffff0000u), __uint_as_float(u[j] & 0xffff0000u));
    y[j] = pack_bf16x2(lo, hi);
  }
  *reinterpret_cast<u32x4*>(out + n * inter + c) = y;
}

}  // namespace

namespace pyre {

bool add_rmsnorm_vec(float* resid, const void* delta, int delta_dt, int n_partials, long partial_stride,
                     const void* gain, int gain_dt, void* out, int out_dt, const int* rows, int n,
                     int hidden, float eps, hipStream_t stream) {
  if (hidden % 4 || hidden > 4 * 256 * kNormMaxVec || (delta && partial_stride % 4)) return false;
  // Which variant runs depends on the number of rows; what it computes does not (see the kernel).
  const bool wide = hidden > 1024;
  const bool few = n <= 128 && wide;  // a decode step: spread each row over more threads
#define PYRE_NORM_LAUNCH(THREADS, VIRT, STREAM)                                                                      \
  hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TD, TG, TO, THREADS, VIRT, STREAM>), dim3(n), dim3(THREADS), 0, stream, \
                     resid, static_cast<const TD*>(delta), n_partials, static_cast<size_t>(partial_stride),          \
                     static_cast<const TG*>(gain), static_cast<TO*>(out), rows, hidden, eps)
  PYRE_DISPATCH(delta_dt, TD, PYRE_DISPATCH(gain_dt, TG, PYRE_DISPATCH(out_dt, TO, {
    const bool many = n >= 512;  // more bytes than the caches keep for the next kernel
    if (few) PYRE_NORM_LAUNCH(1024, 1, false);
    else if (wide && many) PYRE_NORM_LAUNCH(256, 4, true);
    else if (wide) PYRE_NORM_LAUNCH(256, 4, false);
    else if (many) PYRE_NORM_LAUNCH(256, 1, true);
    else PYRE_NORM_LAUNCH(256, 1, false);
  })));
#undef PYRE_NORM_LAUNCH
  return true;
}

bool rope_kv_write_vec(const void* qkv, int qkv_dt, int n_partials, long partial_stride, const void* bias,
                       int bias_dt, void* q_out, int q_dt, void* k_cache, void* v_cache, int cache_dt,
                       const float* cos_t, const float* sin_t, int rotary_dim, const int* positions,
                       const int* slots, int n, int nq, int nkv, int hd, int page_size, int write_kv,
                       hipStream_t stream) {
  if (rotary_dim != hd || hd % 8 || partial_stride % 4 || (write_kv && q_dt != cache_dt)) return false;
  const int items = (nq + nkv) * (hd / 8) + nkv * (hd / 4);
  const dim3 grid(n, (items + 255) / 256);
  if (grid.y > 65535) return false;
#define PYRE_ROPE_LAUNCH(STREAM)                                                                                   \
  PYRE_DISPATCH(qkv_dt, TI, PYRE_DISPATCH(q_dt, TC,                                                               \
      hipLaunchKernelGGL((rope_kv_write_vec_kernel<TI, TC, STREAM>), grid, dim3(256), 0, stream,                  \
                         static_cast<const TI*>(qkv), n_partials, static_cast<size_t>(partial_stride), bias,      \
                         bias_dt, static_cast<TC*>(q_out), static_cast<TC*>(k_cache),                             \
                         static_cast<TC*>(v_cache), cos_t, sin_t, positions, slots, nq, nkv, hd, page_size,       \
                         write_kv)))
  if (n >= 512) {
    PYRE_ROPE_LAUNCH(true);
  } else {
    PYRE_ROPE_LAUNCH(false);
  }
#undef PYRE_ROPE_LAUNCH
  return true;
}

bool silu_mul_vec(const void* gu, int gu_dt, int n_partials, long partial_stride, void* out, int out_dt,
                  int n, int inter, hipStream_t stream) {
  if (inter % 4 || partial_stride % 4) return false;
  if (gu_dt == kBF16 && out_dt == kBF16 && n_partials == 1 && inter % 8 == 0 && n > 128 &&
      reinterpret_cast<uintptr_t>(gu) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const size_t total8 = static_cast<size_t>(n) * (inter / 8);
    hipLaunchKernelGGL(silu_mul_stream_kernel, dim3((total8 + 255) / 256), dim3(256), 0, stream,
                       static_cast<const bf16*>(gu), static_cast<bf16*>(out), total8, inter);
    return true;
  }
  const size_t total4 = static_cast<size_t>(n) * (inter / 4);
  PYRE_DISPATCH(gu_dt, TI, PYRE_DISPATCH(out_dt, TO,
      hipLaunchKernelGGL((silu_mul_vec_kernel<TI, TO>), dim3((total4 + 255) / 256), dim3(256), 0, stream,
                         static_cast<const TI*>(gu), n_partials, static_cast<size_t>(partial_stride),
                         static_cast<TO*>(out), total4, inter)));
  return true;
}

}  // namespace pyre
