// Four elements at a time for the row kernels and for whoever finishes a product's partial sums
// himself: loads and stores of four float32 or bfloat16 values, and the sum of a product's partial
// sums in their fixed order.
#pragma once

#include "pyre_common.h"

namespace pyre {

template <typename T> struct Vec4;
template <> struct Vec4<float> {
  static __device__ inline float4 load(const float* p) { return *reinterpret_cast<const float4*>(p); }
  static __device__ inline void store(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
};
template <> struct Vec4<bf16> {
  static __device__ inline float4 load(const bf16* p) {
    const uint2 u = *reinterpret_cast<const uint2*>(p);
    float4 v;
    v.x = __uint_as_float(u.x << 16);
    v.y = __uint_as_float(u.x & 0xffff0000u);
    v.z = __uint_as_float(u.y << 16);
    v.w = __uint_as_float(u.y & 0xffff0000u);
    return v;
  }
  static __device__ inline void store(bf16* p, float4 v) {
    uint2 u;
    u.x = pack_bf16x2(v.x, v.y);
    u.y = pack_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = u;
  }
};

__device__ inline float4 add4(float4 a, float4 b) { return float4{a.x + b.x, a.y + b.y, a.z + b.z, a.w + b.w}; }

// p[0] + p[1] + ... + p[n - 1] (in that order) of the float4 at `src` in each of n partial sums that
// lie `stride` elements apart. Up to kAtOnce loads are in flight together: a kernel that only
// passes a few rows on spends its time waiting for loads, one round trip after the other.
constexpr int kAtOnce = 12;
template <typename T>
__device__ inline float4 sum_partials4(const T* src, size_t stride, int n) {
  float4 v[kAtOnce];
#pragma unroll
  for (int p = 0; p < kAtOnce; ++p)
    if (p < n) v[p] = Vec4<T>::load(src + p * stride);
  float4 s = v[0];
#pragma unroll
  for (int p = 1; p < kAtOnce; ++p)
    if (p < n) s = add4(s, v[p]);
  for (int p = kAtOnce; p < n; ++p) s = add4(s, Vec4<T>::load(src + p * stride));
  return s;
}

}  // namespace pyre
