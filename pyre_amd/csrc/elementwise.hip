// Embedding lookup, fused residual-add + RMSNorm, rotary + cache write, SiLU-gate
// and the plain reduction of split-K partial sums. All arithmetic is fp32; the
// only roundings are the stores to a 16-bit output.
#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec.h"

using namespace pyre;

// ---------------------------------------------------------------------------
// Embedding: out[n, :] = float(table[ids[n], :])           (pyre/model.py:196)
// ---------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int hidden) {
  const int n = blockIdx.x;
  const T* row = table + static_cast<size_t>(ids[n]) * hidden;
  float* o = out + static_cast<size_t>(n) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = to_float(row[i]);
}

extern "C" int pyre_embed(const void* table, int table_dt, const int* ids, float* out, int n,
                          int hidden, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(table_dt), "embed: unknown table dtype %d", table_dt);
  PYRE_REQUIRE(n >= 0 && hidden > 0, "embed: bad sizes n=%d hidden=%d", n, hidden);
  if (n == 0) return 0;
  PYRE_DISPATCH(table_dt, T,
                hipLaunchKernelGGL(embed_kernel<T>, dim3(n), dim3(256), 0, stream,
                                   static_cast<const T*>(table), ids, out, hidden));
  return check_launch("embed");
}

// ---------------------------------------------------------------------------
// resid += sum_p delta[p] (+ bias);  out = resid * rsqrt(mean(resid^2) + eps) * gain
// (pyre/model.py:33-38 for the norm, :151-152 for the residual sums).
// With `rows` the kernel norms only the listed rows into a dense output and
// leaves `resid` untouched: the final norm before the head needs no more.
// ---------------------------------------------------------------------------
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const void* __restrict__ delta,
                                   int delta_dt, int n_partials, size_t partial_stride,
                                   const void* __restrict__ bias, int bias_dt,
                                   const void* __restrict__ gain, int gain_dt,
                                   void* __restrict__ out, int out_dt, const int* __restrict__ rows,
                                   int hidden, float eps) {
  __shared__ float scratch[16];
  const int r_out = blockIdx.x;
  const int r_in = rows ? rows[r_out] : r_out;
  float* x = resid + static_cast<size_t>(r_in) * hidden;
  const size_t drow = static_cast<size_t>(r_in) * hidden;

  auto value = [&](int i) {
    float v = x[i];
    if (delta) {
      float d = 0.f;
      for (int p = 0; p < n_partials; ++p) d += load_as_float(delta, delta_dt, p * partial_stride + drow + i);
      if (bias) d += load_as_float(bias, bias_dt, i);
      v += d;
    }
    return v;
  };

  float ss = 0.f;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    const float v = value(i);
    if (!rows && delta) x[i] = v;
    ss += v * v;
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / static_cast<float>(hidden) + eps);
  const size_t orow = static_cast<size_t>(r_out) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) {
    // Without `rows` the sum was stored above and is read back; with `rows` it is
    // formed again in the same order, so both passes see the same value.
    const float v = (!rows && delta) ? x[i] : value(i);
    store_from_float(out, out_dt, orow + i, v * inv * load_as_float(gain, gain_dt, i));
  }
}

extern "C" int pyre_add_rmsnorm(float* resid, const void* delta, int delta_dt, int n_partials,
                                long partial_stride, const void* bias, int bias_dt,
                                const void* gain, int gain_dt, void* out, int out_dt,
                                const int* rows, int n, int hidden, float eps,
                                hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(gain_dt) && known_dtype(out_dt), "add_rmsnorm: unknown dtype");
  PYRE_REQUIRE(!delta || (known_dtype(delta_dt) && n_partials >= 1),
               "add_rmsnorm: bad delta (dtype %d, partials %d)", delta_dt, n_partials);
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "add_rmsnorm: unknown bias dtype");
  PYRE_REQUIRE(n >= 0 && hidden > 0 && eps > 0.f, "add_rmsnorm: bad sizes n=%d hidden=%d", n, hidden);
  if (n == 0) return 0;
  if (!bias && add_rmsnorm_vec(resid, delta, delta_dt, delta ? n_partials : 0, partial_stride, gain, gain_dt,
                               out, out_dt, rows, n, hidden, eps, stream))
    return check_launch("add_rmsnorm");
  hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(n), dim3(256), 0, stream, resid, delta, delta_dt,
                     n_partials, static_cast<size_t>(partial_stride), bias, bias_dt, gain, gain_dt,
                     out, out_dt, rows, hidden, eps);
  return check_launch("add_rmsnorm");
}

// ---------------------------------------------------------------------------
// Rotary positions and the cache write, fused with the reduction of the fused
// q/k/v projection (partials + bias). One block per token.
//   q'[j]        = q[j] cos - q[j+r/2] sin,  q'[j+r/2] = q[j+r/2] cos + q[j] sin
// for j < r/2 (r = rotary_dim), the rest passes through  (pyre/model.py:54-63).
// K goes to its page as [page][kv_head][slot][hd]; V transposed, as
// [page][kv_head][hd][slot], so that the attention kernels read runs of keys.
// ---------------------------------------------------------------------------
template <typename TC>
__global__ void rope_kv_write_kernel(const void* __restrict__ qkv, int qkv_dt, int n_partials,
                                     size_t partial_stride, const void* __restrict__ bias,
                                     int bias_dt, void* __restrict__ q_out, int q_dt,
                                     TC* __restrict__ k_cache, TC* __restrict__ v_cache,
                                     const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                     int rotary_dim, const int* __restrict__ positions,
                                     const int* __restrict__ slots, int nq, int nkv, int hd,
                                     int page_size, int write_kv) {
  const int n = blockIdx.x;
  const int width = (nq + 2 * nkv) * hd;
  const size_t in_row = static_cast<size_t>(n) * width;
  const int pos = positions[n];
  const int half = rotary_dim / 2;
  const int slot = write_kv ? slots[n] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const bool tail = write_kv && ends_its_page_run(slots, n, gridDim.x, slot, page_size);

  auto value = [&](int col) {
    float v = 0.f;
    for (int p = 0; p < n_partials; ++p) v += load_as_float(qkv, qkv_dt, p * partial_stride + in_row + col);
    if (bias) v += load_as_float(bias, bias_dt, col);
    return v;
  };

  // Items: for every q and k head the r/2 rotated pairs and the hd-r untouched
  // elements; for every v head its hd elements.
  const int per_head = half + (hd - rotary_dim);
  const int n_rot_items = (nq + nkv) * per_head;
  const int n_items = n_rot_items + nkv * hd;
  for (int it = threadIdx.x; it < n_items; it += blockDim.x) {
    if (it < n_rot_items) {
      const int head = it / per_head, j = it % per_head;
      const int base = head * hd;
      float a, b = 0.f;
      int ia, ib = -1;
      if (j < half) {
        ia = j;
        ib = j + half;
        const float x1 = value(base + ia), x2 = value(base + ib);
        const float c = cos_t[static_cast<size_t>(pos) * half + j];
        const float s = sin_t[static_cast<size_t>(pos) * half + j];
        rotate_pair(x1, x2, c, s, a, b);
      } else {
        ia = rotary_dim + (j - half);
        a = value(base + ia);
      }
      if (head < nq) {
        const size_t o = static_cast<size_t>(n) * nq * hd + base;
        store_from_float(q_out, q_dt, o + ia, a);
        if (ib >= 0) store_from_float(q_out, q_dt, o + ib, b);
      } else if (slot >= 0) {
        const int kvh = head - nq;
        TC* dst = k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + off) * hd;
        dst[ia] = from_float<TC>(a);
        if (ib >= 0) dst[ib] = from_float<TC>(b);
      }
    } else if (slot >= 0) {
      const int e = it - n_rot_items;
      const int kvh = e / hd, d = e % hd;
      const float v = value((nq + nkv) * hd + e);
      TC* row = v_cache + ((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size;
      row[off] = from_float<TC>(v);
      if (tail) zero_tail(row, off + 1, page_size);  // nothing of the page's previous owner stays behind the last key
    }
  }
}

extern "C" int pyre_rope_kv_write(const void* qkv, int qkv_dt, int n_partials, long partial_stride,
                                  const void* bias, int bias_dt, void* q_out, int q_dt,
                                  void* k_cache, void* v_cache, int cache_dt, const float* cos_t,
                                  const float* sin_t, int rotary_dim, const int* positions,
                                  const int* slots, int n, int nq, int nkv, int hd, int page_size,
                                  int write_kv, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(qkv_dt) && known_dtype(q_dt) && known_dtype(cache_dt),
               "rope_kv_write: unknown dtype");
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "rope_kv_write: unknown bias dtype");
  PYRE_REQUIRE(n_partials >= 1, "rope_kv_write: n_partials=%d", n_partials);
  PYRE_REQUIRE(nq > 0 && nkv > 0 && hd > 0 && page_size > 0, "rope_kv_write: bad sizes");
  PYRE_REQUIRE(rotary_dim >= 0 && rotary_dim <= hd && rotary_dim % 2 == 0,
               "rope_kv_write: rotary_dim %d must be even and at most head_dim %d", rotary_dim, hd);
  PYRE_REQUIRE(rotary_dim == 0 || (cos_t && sin_t), "rope_kv_write: rotary tables missing");
  if (n <= 0) return 0;
  if (rope_kv_write_vec(qkv, qkv_dt, n_partials, partial_stride, bias, bias_dt, q_out, q_dt, k_cache, v_cache,
                        write_kv ? cache_dt : q_dt, cos_t, sin_t, rotary_dim, positions, slots, n, nq, nkv, hd,
                        page_size, write_kv, stream))
    return check_launch("rope_kv_write");
  PYRE_DISPATCH(cache_dt, TC,
                hipLaunchKernelGGL(rope_kv_write_kernel<TC>, dim3(n), dim3(256), 0, stream, qkv,
                                   qkv_dt, n_partials, static_cast<size_t>(partial_stride), bias,
                                   bias_dt, q_out, q_dt, static_cast<TC*>(k_cache),
                                   static_cast<TC*>(v_cache), cos_t, sin_t, rotary_dim, positions,
                                   slots, nq, nkv, hd, page_size, write_kv));
  return check_launch("rope_kv_write");
}

// ---------------------------------------------------------------------------
// act[n, i] = silu(gate[n, i]) * up[n, i], gate = gu[:, :I], up = gu[:, I:]
// (pyre/model.py:139); silu(z) = z / (1 + exp(-z)).
// ---------------------------------------------------------------------------
__global__ void silu_mul_kernel(const void* __restrict__ gu, int gu_dt, int n_partials,
                                size_t partial_stride, void* __restrict__ out, int out_dt,
                                size_t total, int inter) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const size_t n = i / inter, c = i % inter;
  const size_t gi = n * 2 * inter + c, ui = gi + inter;
  float g = 0.f, u = 0.f;
  for (int p = 0; p < n_partials; ++p) {
    g += load_as_float(gu, gu_dt, p * partial_stride + gi);
    u += load_as_float(gu, gu_dt, p * partial_stride + ui);
  }
  store_from_float(out, out_dt, i, g / (1.f + expf(-g)) * u);
}

extern "C" int pyre_silu_mul(const void* gu, int gu_dt, int n_partials, long partial_stride,
                             void* out, int out_dt, int n, int inter, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(gu_dt) && known_dtype(out_dt), "silu_mul: unknown dtype");
  PYRE_REQUIRE(n_partials >= 1 && inter > 0, "silu_mul: bad sizes");
  if (n <= 0) return 0;
  if (silu_mul_vec(gu, gu_dt, n_partials, partial_stride, out, out_dt, n, inter, stream))
    return check_launch("silu_mul");
  const size_t total = static_cast<size_t>(n) * inter;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, gu, gu_dt,
                     n_partials, static_cast<size_t>(partial_stride), out, out_dt, total, inter);
  return check_launch("silu_mul");
}

// ---------------------------------------------------------------------------
// out[n, c] = sum_p in[p][n, c] (+ bias[c]): for consumers that do not fuse the
// reduction of split-K partial sums into their own kernel.
// ---------------------------------------------------------------------------
__global__ void reduce_partials_kernel(const void* __restrict__ in, int in_dt, int n_partials,
                                       size_t partial_stride, const void* __restrict__ bias,
                                       int bias_dt, void* __restrict__ out, int out_dt,
                                       size_t total, int width) {
  const size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float v = 0.f;
  for (int p = 0; p < n_partials; ++p) v += load_as_float(in, in_dt, p * partial_stride + i);
  if (bias) v += load_as_float(bias, bias_dt, i % width);
  store_from_float(out, out_dt, i, v);
}

extern "C" int pyre_reduce_partials(const void* in, int in_dt, int n_partials, long partial_stride,
                                    const void* bias, int bias_dt, void* out, int out_dt, int n,
                                    int width, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(in_dt) && known_dtype(out_dt), "reduce_partials: unknown dtype");
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "reduce_partials: unknown bias dtype");
  PYRE_REQUIRE(n_partials >= 1 && width > 0, "reduce_partials: bad sizes");
  if (n <= 0) return 0;
  const size_t total = static_cast<size_t>(n) * width;
  hipLaunchKernelGGL(reduce_partials_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, in,
                     in_dt, n_partials, static_cast<size_t>(partial_stride), bias, bias_dt, out,
                     out_dt, total, width);
  return check_launch("reduce_partials");
}

// ---------------------------------------------------------------------------
// Fill utility: sets whole rows of a [outer, rows, row_elems] tensor to one bit pattern.
// It zeroes a request's state slot at admission and, in the debug mode that poisons freed
// memory, writes NaN over pages and slots that went back to their pool. The row ids come
// from the host by value, so no upload is needed.
// ---------------------------------------------------------------------------
namespace {
constexpr int kFillIds = 64;
struct FillIds { int v[kFillIds]; };

template <typename U>
__global__ __launch_bounds__(256) void fill_rows_kernel(U* __restrict__ base, size_t outer_stride, size_t row_elems,
                                                        FillIds ids, U pattern) {
  U* row = base + blockIdx.z * outer_stride + static_cast<size_t>(ids.v[blockIdx.y]) * row_elems;
  for (size_t i = static_cast<size_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < row_elems;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    row[i] = pattern;
}
}  // namespace

extern "C" int pyre_fill_rows(void* base, int elem_bytes, long outer_stride, int n_outer, int n_rows, long row_elems,
                              const int* ids_host, int n_ids, unsigned pattern, hipStream_t stream) {
  PYRE_REQUIRE(elem_bytes == 2 || elem_bytes == 4, "fill_rows: elements of %d bytes", elem_bytes);
  PYRE_REQUIRE(n_outer >= 1 && n_outer <= 65535 && row_elems >= 1 && outer_stride >= static_cast<long>(n_rows) * row_elems,
               "fill_rows: bad sizes");
  for (int i = 0; i < n_ids; ++i)
    PYRE_REQUIRE(ids_host[i] >= 0 && ids_host[i] < n_rows, "fill_rows: row %d is outside 0..%d", ids_host[i], n_rows - 1);
  const unsigned bx = static_cast<unsigned>(row_elems / 256 < 1 ? 1 : (row_elems / 256 > 64 ? 64 : row_elems / 256));
  for (int done = 0; done < n_ids; done += kFillIds) {
    FillIds ids;
    const int now = n_ids - done < kFillIds ? n_ids - done : kFillIds;
    for (int i = 0; i < kFillIds; ++i) ids.v[i] = ids_host[done + (i < now ? i : 0)];
    const dim3 grid(bx, now, n_outer);
    if (elem_bytes == 4)
      hipLaunchKernelGGL(fill_rows_kernel<uint32_t>, grid, dim3(256), 0, stream, static_cast<uint32_t*>(base),
                         static_cast<size_t>(outer_stride), static_cast<size_t>(row_elems), ids, pattern);
    else
      hipLaunchKernelGGL(fill_rows_kernel<uint16_t>, grid, dim3(256), 0, stream, static_cast<uint16_t*>(base),
                         static_cast<size_t>(outer_stride), static_cast<size_t>(row_elems), ids,
                         static_cast<uint16_t>(pattern));
  }
  return check_launch("fill_rows");
}
