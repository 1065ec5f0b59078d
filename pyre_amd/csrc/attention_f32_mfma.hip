// Causal (optionally windowed) attention of prompt portions over the paged cache in true
// float32 on the matrix cores (v_mfma_f32_32x32x2_f32: float32 operands, products and sums):
// the 32-bit path's attention for requests that bring more than one token. Single tokens stay
// with attention_generic.hip, whose one block per (token, head) cannot use a 32-column tile.
//
//   scores = (q k^T) * scale, masked to lo..pos       (pyre/model.py:109-120)
//   probs  = softmax(scores), out = probs v            (pyre/model.py:122-123)
//
// A tile is up to 32 consecutive tokens of one request (tiles[i] = first token in the flat
// batch, count). A block of four waves takes four query heads of one key/value head over
// the same tile: the keys and values of a chunk of 32 keys are staged in LDS once per block
// (K as stored, V transposed back: [d][key]), each wave multiplies them with its own head.
// As in attention_mfma.hip the transposed problem is computed, so that the scores come out
// in the layout the second product wants them in:
//   S^T[key, token]  = sum_d K[key, d] Q[token, d]      A = K (LDS), B = Q^T (registers)
//   O^T[d, token]   += sum_key V^T[d, key] P^T[key, token]   A = V^T (LDS), B = P^T = the lane's
//                                                           own sixteen scores, one per step
// Step s of the second product takes key 8 (s / 4) + (s % 4) of the chunk in lanes 0..31 and
// key 8 (s / 4) + 4 + (s % 4) in lanes 32..63: exactly the keys whose scores those lanes hold
// in accumulator element s. Chunks start at multiples of 32 keys, so the order of every sum
// of a token depends on its own bounds (lo, pos) alone, not on the tile it is in or on what
// else is in the step.
#include <type_traits>

#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;
constexpr int kKeys = 32;

// HDP: the head size rounded up to a multiple of 32 (the rest is zeros).
template <int HDP>
__global__ __launch_bounds__(256) void attn_prefill_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k_cache, const float* __restrict__ v_cache,
    float* __restrict__ out, const int* __restrict__ tiles, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride, int nq, int nkv,
    int hd, int page_size, float scale, int window) {
  __shared__ float Ks[kKeys][HDP + 1];   // rows on distinct banks for the lanes of a half-wave
  __shared__ float Vt[HDP][kKeys + 1];
  __shared__ int page_s[kKeys];          // the page of each key of the chunk, -1 if it is not there
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, h = lane >> 5, c = lane & 31;
  const int n_rep = nq / nkv, hgroups = (n_rep + 3) / 4;
  const int kvh = blockIdx.y / hgroups, hin = (blockIdx.y % hgroups) * 4 + wave;
  const bool active = hin < n_rep;  // a wave without a head still helps loading
  const int head = kvh * n_rep + (active ? hin : 0);
  const int t0 = tiles[2 * blockIdx.x], ntok = tiles[2 * blockIdx.x + 1];
  if (ntok <= 0) return;
  const int pos0 = positions[t0];
  const int* table = block_table + static_cast<size_t>(seq_of_token[t0]) * table_stride;

  // Column c of this wave: token t0 + c, which sees keys lo..hi. Columns past the tile's end
  // compute on zeros over the first token's keys and are not stored.
  const bool live = active && c < ntok;
  const int hi = c < ntok ? pos0 + c : pos0;
  const int lo = window > 0 ? max(0, hi - window + 1) : 0;
  float qr[HDP / 2];  // Q[token c][d = 2 s + h]
#pragma unroll
  for (int s = 0; s < HDP / 2; ++s) {
    const int d = 2 * s + h;
    qr[s] = live && d < hd ? q[(static_cast<size_t>(t0 + c) * nq + head) * hd + d] : 0.f;
  }
  f32x16 o[HDP / 32];
#pragma unroll
  for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m = -INFINITY, l = 0.f;  // l: this lane's share of the column's sum (its sixteen keys of every chunk)

  const int lo_all = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int hi_all = pos0 + ntok - 1;
  for (int chunk = lo_all / kKeys; chunk <= hi_all / kKeys; ++chunk) {
    const int key0 = chunk * kKeys;
    __syncthreads();  // the previous chunk has been read by every wave
    if (tid < kKeys) {
      const int key = key0 + tid, entry = key / page_size;
      page_s[tid] = key <= hi_all && entry < table_stride ? table[entry] : -1;
    }
    __syncthreads();
    for (int i = tid; i < kKeys * HDP; i += 256) {  // K: d fastest, as it lies in the cache
      const int key = i / HDP, d = i % HDP, page = page_s[key];
      float v = 0.f;
      if (page >= 0 && d < hd)
        v = k_cache[((static_cast<size_t>(page) * nkv + kvh) * page_size + (key0 + key) % page_size) * hd + d];
      Ks[key][d] = v;
    }
    for (int i = tid; i < kKeys * HDP; i += 256) {  // V: the key fastest, as the cache stores it transposed
      const int d = i / kKeys, key = i % kKeys, page = page_s[key];
      float v = 0.f;
      if (page >= 0 && d < hd)
        v = v_cache[((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size + (key0 + key) % page_size];
      Vt[d][key] = v;
    }
    __syncthreads();
    if (!active) continue;

    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
    for (int st = 0; st < HDP / 2; ++st) s = __builtin_amdgcn_mfma_f32_32x32x2f32(Ks[c][2 * st + h], qr[st], s, 0, 0, 0);

    // element i of s: key key0 + 8 (i / 4) + 4 h + i % 4, token c
    float mx = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int kk = 8 * (i >> 2) + 4 * h + (i & 3), key = key0 + kk;
      s[i] = (key < lo || key > hi || page_s[kk] < 0) ? -INFINITY : s[i] * scale;
      mx = fmaxf(mx, s[i]);
    }
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // a column without a visible key so far
    const float alpha = expf(m - m_use);
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      s[i] = expf(s[i] - m_use);
      sum += s[i];
    }
    l = l * alpha + sum;
#pragma unroll
    for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
#pragma unroll
    for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
      for (int st = 0; st < 16; ++st)
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(Vt[32 * dt + c][8 * (st >> 2) + 4 * h + (st & 3)], s[st], o[dt], 0, 0, 0);
  }

  if (!active) return;
  l += __shfl_xor(l, 32, 64);
  if (c >= ntok) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  float* dst = out + (static_cast<size_t>(t0 + c) * nq + head) * hd;
  // element 4 i + j of o[dt]: d = 32 dt + 8 i + 4 h + j
#pragma unroll
  for (int dt = 0; dt < HDP / 32; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int d = 32 * dt + 8 * (i >> 2) + 4 * h + (i & 3);
      if (d < hd) dst[d] = o[dt][i] * inv;
    }
}

}  // namespace

extern "C" int pyre_attn_prefill_f32(const float* q, float* out, const float* k_cache, const float* v_cache,
                                     const int* tiles, int n_tiles, const int* positions, const int* seq_of_token,
                                     const int* block_table, int table_stride, int nq, int nkv, int hd, int page_size,
                                     float scale, int window, hipStream_t stream) {
  PYRE_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attn_prefill_f32: %d query heads do not divide over %d kv heads", nq, nkv);
  PYRE_REQUIRE(hd > 0 && hd <= 256, "attn_prefill_f32: head_dim %d is outside 1..256", hd);
  PYRE_REQUIRE(page_size > 0 && table_stride > 0, "attn_prefill_f32: bad page geometry");
  if (n_tiles <= 0) return 0;
  const int hgroups = (nq / nkv + 3) / 4;
  PYRE_REQUIRE(nkv * hgroups <= 65535, "attn_prefill_f32: grid too large");
  const dim3 grid(n_tiles, nkv * hgroups);
#define PYRE_F32_ATTN(HDP)                                                                                        \
  hipLaunchKernelGGL(attn_prefill_f32_kernel<HDP>, grid, dim3(256), 0, stream, q, k_cache, v_cache, out, tiles,    \
                     positions, seq_of_token, block_table, table_stride, nq, nkv, hd, page_size, scale, window)
  switch ((hd + 31) / 32) {
    case 1: PYRE_F32_ATTN(32); break;
    case 2: PYRE_F32_ATTN(64); break;
    case 3: PYRE_F32_ATTN(96); break;
    case 4: PYRE_F32_ATTN(128); break;
    case 5: PYRE_F32_ATTN(160); break;
    case 6: PYRE_F32_ATTN(192); break;
    case 7: PYRE_F32_ATTN(224); break;
    default: PYRE_F32_ATTN(256); break;
  }
#undef PYRE_F32_ATTN
  return check_launch("attn_prefill_f32");
}
