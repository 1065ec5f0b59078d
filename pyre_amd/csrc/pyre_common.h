// Shared helpers for the gfx950 kernels: element types, conversions, reductions,
// error reporting. Everything here is device code for 64-wide wavefronts.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

namespace pyre {

constexpr int kWave = 64;

// Element type codes shared with the Python binding.
enum DType : int { kF32 = 0, kBF16 = 1 };

// bfloat16 as its raw 16 bits; conversions are explicit so that every rounding
// in a kernel is visible where it happens.
struct bf16 {
  uint16_t bits;
};

__host__ __device__ inline float to_float(float v) { return v; }
__host__ __device__ inline float to_float(bf16 v) {
  union { uint32_t u; float f; } x;
  x.u = static_cast<uint32_t>(v.bits) << 16;
  return x.f;
}

typedef __bf16 hw_bf16x2 __attribute__((ext_vector_type(2)));
typedef float hw_f32x2 __attribute__((ext_vector_type(2)));

// Two floats to two bfloat16 in one word (low half first), round to nearest even:
// one v_cvt_pk_bf16_f32 on the device.
__device__ inline uint32_t pack_bf16x2(float lo, float hi) {
  const hw_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, hw_bf16x2));
}

// Round to nearest, ties to even; NaN stays NaN.
__host__ __device__ inline uint16_t bf16_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return static_cast<uint16_t>(pack_bf16x2(f, 0.f) & 0xffffu);
#endif
  union { uint32_t u; float f; } x;
  x.f = f;
  if ((x.u & 0x7fffffffu) > 0x7f800000u) return static_cast<uint16_t>((x.u >> 16) | 0x40u);
  x.u += 0x7fffu + ((x.u >> 16) & 1u);
  return static_cast<uint16_t>(x.u >> 16);
}

// One rotary pair turned by the angle with cosine c and sine s (pyre/model.py:54-63), with
// explicit fused multiply-adds: the same roundings in every kernel that rotates.
__device__ inline void rotate_pair(float x1, float x2, float c, float s, float& a, float& b) {
  a = fmaf(x1, c, -(x2 * s));
  b = fmaf(x2, c, x1 * s);
}

// The attention kernels on the matrix cores load whole chunks of values and weight the keys
// that a query does not see with an exact 0, which only a finite value survives. The slots of a
// request's last page after its last key hold what the page's previous owner left there (NaN
// and Inf included), so whoever writes a step's last token into a page also zeroes the values
// of the slots after it: what follows a request's last key in its page is always zero.
//   ends_its_page_run: token n of a step of `count` tokens, written to `slot`, is the last one
//                      that the step writes into its page (the next token, if there is one, does
//                      not take the next slot), and the page has slots after it;
//   zero_tail:         row[from .. to) = 0 in as few stores as the alignment allows.
__device__ inline bool ends_its_page_run(const int* slots, int n, int count, int slot, int page_size) {
  return slot >= 0 && slot % page_size + 1 < page_size && (n + 1 >= count || slots[n + 1] != slot + 1);
}
template <typename T>
__device__ inline void zero_tail(T* row, int from, int to) {
  static_assert(sizeof(T) == 2 || sizeof(T) == 4, "cache elements of two or four bytes");
  char* p = reinterpret_cast<char*>(row + from);
  char* const end = reinterpret_cast<char*>(row + to);
  while (p < end) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    const size_t left = static_cast<size_t>(end - p);
    if (a % 16 == 0 && left >= 16) {
      *reinterpret_cast<uint4*>(p) = uint4{0u, 0u, 0u, 0u};
      p += 16;
    } else if (a % 8 == 0 && left >= 8) {
      *reinterpret_cast<uint2*>(p) = uint2{0u, 0u};
      p += 8;
    } else if (a % 4 == 0 && left >= 4) {
      *reinterpret_cast<uint32_t*>(p) = 0u;
      p += 4;
    } else {
      *reinterpret_cast<uint16_t*>(p) = 0;
      p += 2;
    }
  }
}

template <typename T> __host__ __device__ inline T from_float(float v);
template <> __host__ __device__ inline float from_float<float>(float v) { return v; }
template <> __host__ __device__ inline bf16 from_float<bf16>(float v) {
  bf16 r;
  r.bits = bf16_bits(v);
  return r;
}

// Read element i of an array whose element type is only known at run time.
__device__ inline float load_as_float(const void* p, int dt, size_t i) {
  return dt == kF32 ? static_cast<const float*>(p)[i] : to_float(static_cast<const bf16*>(p)[i]);
}
__device__ inline void store_from_float(void* p, int dt, size_t i, float v) {
  if (dt == kF32) static_cast<float*>(p)[i] = v;
  else static_cast<bf16*>(p)[i] = from_float<bf16>(v);
}

__device__ inline float wave_sum(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ inline float wave_max(float v) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

// Block-wide reductions for blocks of up to 1024 threads (16 waves). `scratch`
// is 16 floats of LDS. Every thread receives the result; the order of the
// additions is fixed by the thread layout alone.
__device__ inline float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int w = threadIdx.x / kWave, nw = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[w] = v;
  __syncthreads();
  float t = 0.f;
  for (int i = 0; i < nw; ++i) t += scratch[i];
  return t;
}
__device__ inline float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int w = threadIdx.x / kWave, nw = (blockDim.x + kWave - 1) / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[w] = v;
  __syncthreads();
  float t = scratch[0];
  for (int i = 1; i < nw; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

// ---- host side -------------------------------------------------------------

// The last error of this thread, returned to Python by pyre_last_error().
char* error_buffer();

// Compute units of the current device (runtime.hip); launch shapes that are made to fill the
// chip in one round of blocks follow it.
constexpr int kDefaultUnits = 256;  // an MI355X
int compute_units();

inline int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(error_buffer(), 512, fmt, ap);
  va_end(ap);
  return 1;
}

inline int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail("%s: %s", what, hipGetErrorString(e));
  return 0;
}

inline bool known_dtype(int dt) { return dt == kF32 || dt == kBF16; }

}  // namespace pyre

#define PYRE_REQUIRE(cond, ...) \
  do {                          \
    if (!(cond)) return pyre::fail(__VA_ARGS__); \
  } while (0)

// Calls `body` with `T` bound to the element type that `dt` names.
#define PYRE_DISPATCH(dt, T, ...)                         \
  do {                                                    \
    if ((dt) == pyre::kF32) { using T = float; __VA_ARGS__; } \
    else { using T = pyre::bf16; __VA_ARGS__; }           \
  } while (0)
