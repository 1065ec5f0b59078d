// Vectorised row kernels (elementwise_vec.hip): each returns false without
// launching when the case is not one it takes; the caller then runs the general kernel.
#pragma once

#include <hip/hip_runtime.h>

namespace pyre {

bool add_rmsnorm_vec(float* resid, const void* delta, int delta_dt, int n_partials, long partial_stride,
                     const void* gain, int gain_dt, void* out, int out_dt, const int* rows, int n,
                     int hidden, float eps, hipStream_t stream);

bool rope_kv_write_vec(const void* qkv, int qkv_dt, int n_partials, long partial_stride, const void* bias,
                       int bias_dt, void* q_out, int q_dt, void* k_cache, void* v_cache, int cache_dt,
                       const float* cos_t, const float* sin_t, int rotary_dim, const int* positions,
                       const int* slots, int n, int nq, int nkv, int hd, int page_size, int write_kv,
                       hipStream_t stream);

bool silu_mul_vec(const void* gu, int gu_dt, int n_partials, long partial_stride, void* out, int out_dt,
                  int n, int inter, hipStream_t stream);

}  // namespace pyre
