// Causal (optionally windowed) attention of every token of a step over the paged
// cache, for any head size up to 256, any page size, any grouping of heads and
// either element type; all arithmetic fp32. One block per (token, query head, span of keys).
//
//   scores[j] = (q . k_j) * scale      for lo <= j <= pos     (pyre/model.py:109)
//   probs     = softmax(scores)                               (pyre/model.py:122)
//   out       = sum_j probs[j] v_j                            (pyre/model.py:123)
//
// `tokens` (or null: all of them) lists the n tokens of the flat batch to attend for.
// A token at position `pos` sees the keys lo..pos of its request, all read from
// the cache (this step's keys were written before the call), so prompt portions
// and single decoded tokens are the same case. lo = max(0, pos - window + 1) for
// a window, else 0. The keys of a token are taken in spans of 128, one block each (grid.z),
// whose partial results (max, sum, unnormalised output) a second kernel joins in the order of
// the spans; a launch whose block tables hold no more than one span writes the result
// directly. The order of every sum depends on (lo, pos) alone, so the result for a position
// does not depend on how the step was cut or batched.
// This is the 32-bit path's attention and the 16-bit path's fallback; it stands
// where the reference has `forward_paged`'s gather + matmuls (pyre/model.py:274-290)
// and its decode kernel (pyre/kernels/paged_attn.py:26-71).
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;
constexpr int kSpan = 128;     // keys that one block takes, and whose scores are held in LDS
constexpr int kMaxHead = 256;

// Four consecutive elements as one load; p is aligned to four elements.
template <typename T>
__device__ inline void load4(const T* p, float (&v)[4]) {
  struct __attribute__((aligned(4 * sizeof(T)))) Quad { T e[4]; };
  const Quad q = *reinterpret_cast<const Quad*>(p);
#pragma unroll
  for (int u = 0; u < 4; ++u) v[u] = to_float(q.e[u]);
}

// VEC: head size and page size are multiples of four and the caches start on 16 bytes, so
// that keys are read four elements and values four keys at a time. The sums of a score run
// over the elements in their order either way.
template <typename TQ, typename TC, bool VEC>
__global__ __launch_bounds__(kThreads) void attn_generic_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    TQ* __restrict__ out, const int* __restrict__ tokens, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride, int nq, int nkv,
    int hd, int page_size, float scale, int window, float* __restrict__ part) {
  __shared__ float qs[kMaxHead];
  __shared__ float sc[kSpan];
  __shared__ float accs[kThreads];
  __shared__ float scratch[16];

  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (nq / nkv);
  const int pos = positions[n];
  const int* table = block_table + static_cast<size_t>(seq_of_token[n]) * table_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int base = lo + static_cast<int>(blockIdx.z) * kSpan;  // this block's span
  if (base > pos) return;

  for (int d = tid; d < hd; d += kThreads) qs[d] = to_float(q[(static_cast<size_t>(n) * nq + h) * hd + d]);
  __syncthreads();

  // The second product splits the threads into `groups` sets of hd threads;
  // set g takes the keys g, g + groups, ... of a chunk for output element d.
  const int groups = kThreads / hd;  // >= 1 because hd <= 256
  const int g = tid / hd, d = tid % hd;
  const bool active = g < groups;

  float m = -INFINITY, l = 0.f, acc = 0.f;
  {
    const int cnt = min(kSpan, pos - base + 1);
    float lmax = -INFINITY;
    for (int j = tid; j < cnt; j += kThreads) {
      const int key = base + j;
      const int page = table[key / page_size], off = key % page_size;
      float s = -INFINITY;  // a page that is not there (padding rows of a captured step) hides its keys
      if (page >= 0) {
        const TC* kp = k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + off) * hd;
        s = 0.f;
        if (VEC) {
#pragma unroll 8
          for (int e = 0; e < hd; e += 4) {
            float kv[4];
            load4(kp + e, kv);
#pragma unroll
            for (int u = 0; u < 4; ++u) s = fmaf(qs[e + u], kv[u], s);
          }
        } else {
          for (int e = 0; e < hd; ++e) s = fmaf(qs[e], to_float(kp[e]), s);
        }
        s *= scale;
      }
      sc[j] = s;
      lmax = fmaxf(lmax, s);
    }
    m = block_max(lmax, scratch);
    const float m_use = m == -INFINITY ? 0.f : m;
    float lsum = 0.f;
    for (int j = tid; j < cnt; j += kThreads) {
      const float p = expf(sc[j] - m_use);
      sc[j] = p;
      lsum += p;
    }
    l = block_sum(lsum, scratch);  // block_sum's barriers publish sc[]
    if (active && VEC) {  // groups of four keys that lie side by side in a page
#pragma unroll 4
      for (int quad = base / 4 + g; quad <= (base + cnt - 1) / 4; quad += groups) {
        const int key = 4 * quad;
        const int page = table[key / page_size], off = key % page_size;
        if (page < 0) continue;
        float vv[4];
        load4(v_cache + ((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size + off, vv);
#pragma unroll
        for (int u = 0; u < 4; ++u)
          if (key + u >= base && key + u < base + cnt) acc = fmaf(sc[key + u - base], vv[u], acc);
      }
    } else if (active) {
      for (int j = g; j < cnt; j += groups) {
        const int key = base + j;
        const int page = table[key / page_size], off = key % page_size;
        if (page < 0) continue;
        const TC* vp = v_cache + ((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size + off;
        acc = fmaf(sc[j], to_float(*vp), acc);
      }
    }
  }

  accs[tid] = active ? acc : 0.f;
  __syncthreads();
  if (tid < hd) {
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += accs[gg * hd + tid];
    if (part) {  // [token of the list][head][span][hd + 2]: unnormalised output, max, sum
      float* dst = part + ((static_cast<size_t>(blockIdx.x) * nq + h) * gridDim.z + blockIdx.z) * (hd + 2);
      dst[tid] = total;
      if (tid == 0) {
        dst[hd] = m;
        dst[hd + 1] = l;
      }
    } else {
      out[(static_cast<size_t>(n) * nq + h) * hd + tid] = from_float<TQ>(l > 0.f ? total / l : 0.f);
    }
  }
}

// The same for the query heads that share a key/value head, float32 throughout: one block per
// (token, key/value head and group of up to kGroupHeads of its query heads, span of keys), so
// that a span's keys and values are read once for the group and not once per head (a decode
// step's attention is all memory traffic). Every number is computed exactly as the kernel
// above computes it, by the same chain of operations in the same order: a score by one thread
// (the key's, for all heads of the group) over the head's elements in ascending order; a span's sum of probabilities by the same
// reduction over the same layout of threads (key j in lane j % 64 of wave j / 64, the waves'
// sums added in their order); an output element over the keys 4 g, 4 g + 1, ... of its thread's
// set, the sets' sums added in their order. The two kernels give the same bits; this one needs
// head and page sizes that are multiples of four (VEC above).
constexpr int kGroupHeads = 8;

__global__ __launch_bounds__(kThreads) void attn_grouped_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k_cache, const float* __restrict__ v_cache,
    float* __restrict__ out, const int* __restrict__ tokens, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride, int nq, int nkv,
    int hd, int page_size, float scale, int window, float* __restrict__ part) {
  __shared__ __attribute__((aligned(16))) float sc[kGroupHeads][kSpan];
  __shared__ float accs[kGroupHeads][kThreads];
  __shared__ float ml[kGroupHeads][2];  // maximum and sum of each head's span
  __shared__ float scratch[16];

  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, tid = threadIdx.x;
  const int n_rep = nq / nkv, per_kv = (n_rep + kGroupHeads - 1) / kGroupHeads;
  const int kvh = blockIdx.y / per_kv, head0 = kvh * n_rep + (blockIdx.y % per_kv) * kGroupHeads;
  const int nheads = min(kGroupHeads, kvh * n_rep + n_rep - head0);
  const int pos = positions[n];
  const int* table = block_table + static_cast<size_t>(seq_of_token[n]) * table_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int base = lo + static_cast<int>(blockIdx.z) * kSpan;  // this block's span
  if (base > pos) return;
  const int cnt = min(kSpan, pos - base + 1);

  // Scores: thread j < 128 takes key base + j for every head of the group (each row of keys is read by
  // one thread only: a wave's load touches 64 lines, and the address unit's time is what this phase
  // costs). The queries are the same for every lane: they come through scalar loads.
  const int j = tid;
  const float* qg = q + (static_cast<size_t>(n) * nq + head0) * hd;
  float s[kGroupHeads];
#pragma unroll
  for (int h = 0; h < kGroupHeads; ++h) s[h] = -INFINITY;
  if (j < cnt) {
    const int key = base + j;
    const int page = table[key / page_size], off = key % page_size;
    if (page >= 0) {  // a page that is not there (padding rows of a captured step) hides its keys
      const float* kp = k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + off) * hd;
#pragma unroll
      for (int h = 0; h < kGroupHeads; ++h) s[h] = 0.f;
#pragma unroll 8
      for (int e = 0; e < hd; e += 4) {
        float kv[4];
        load4(kp + e, kv);
#pragma unroll
        for (int h = 0; h < kGroupHeads; ++h)
          if (h < nheads) {
#pragma unroll
            for (int u = 0; u < 4; ++u) s[h] = fmaf(qg[h * hd + e + u], kv[u], s[h]);
          }
      }
#pragma unroll
      for (int h = 0; h < kGroupHeads; ++h) s[h] *= scale;
    }
  }
  // Softmax of the span, head by head: the maximum, the probabilities, their sum (key j in lane
  // j % 64 of wave j / 64, the other two waves add zeros).
#pragma unroll
  for (int h = 0; h < kGroupHeads; ++h) {
    if (h >= nheads) break;
    const bool mine = j < cnt;
    const float m = block_max(mine ? s[h] : -INFINITY, scratch);
    const float m_use = m == -INFINITY ? 0.f : m;
    const float p = mine ? expf(s[h] - m_use) : 0.f;
    if (mine) sc[h][j] = p;
    const float l = block_sum(p, scratch);  // its barriers publish sc[h][]
    if (tid == 0) ml[h][0] = m, ml[h][1] = l;
  }

  // Output: set g of hd threads takes the groups of four keys g, g + groups, ... of the span for element d.
  const int groups = kThreads / hd;  // >= 1 because hd <= 256
  const int g = tid / hd, d = tid % hd;
  float acc[kGroupHeads];
#pragma unroll
  for (int h = 0; h < kGroupHeads; ++h) acc[h] = 0.f;
  if (g < groups) {
#pragma unroll 2
    for (int quad = base / 4 + g; quad <= (base + cnt - 1) / 4; quad += groups) {
      const int key = 4 * quad;
      const int page = table[key / page_size], off = key % page_size;
      if (page < 0) continue;
      float vv[4];
      load4(v_cache + ((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size + off, vv);
      if (key >= base && key + 3 < base + cnt && ((key - base) & 3) == 0) {  // the whole group, its probabilities in one read
#pragma unroll
        for (int h = 0; h < kGroupHeads; ++h)
          if (h < nheads) {
            const float4 p = *reinterpret_cast<const float4*>(&sc[h][key - base]);
            acc[h] = fmaf(p.x, vv[0], acc[h]);
            acc[h] = fmaf(p.y, vv[1], acc[h]);
            acc[h] = fmaf(p.z, vv[2], acc[h]);
            acc[h] = fmaf(p.w, vv[3], acc[h]);
          }
        continue;
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (key + u >= base && key + u < base + cnt) {
#pragma unroll
          for (int h = 0; h < kGroupHeads; ++h)
            if (h < nheads) acc[h] = fmaf(sc[h][key + u - base], vv[u], acc[h]);
        }
    }
  }
#pragma unroll
  for (int h = 0; h < kGroupHeads; ++h) accs[h][tid] = g < groups ? acc[h] : 0.f;
  __syncthreads();
  for (int i = tid; i < nheads * hd; i += kThreads) {
    const int h = i / hd, dd = i % hd;
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += accs[h][gg * hd + dd];
    if (part) {  // [token of the list][head][span][hd + 2]: unnormalised output, max, sum
      float* dst = part + ((static_cast<size_t>(blockIdx.x) * nq + head0 + h) * gridDim.z + blockIdx.z) * (hd + 2);
      dst[dd] = total;
      if (dd == 0) {
        dst[hd] = ml[h][0];
        dst[hd + 1] = ml[h][1];
      }
    } else {
      const float l = ml[h][1];
      out[(static_cast<size_t>(n) * nq + head0 + h) * hd + dd] = l > 0.f ? total / l : 0.f;
    }
  }
}

// out = sum_s acc_s e^(m_s - M) / sum_s l_s e^(m_s - M) over the spans that the token has, in their order.
template <typename TQ>
__global__ __launch_bounds__(kThreads) void attn_generic_join_kernel(
    const float* __restrict__ part, TQ* __restrict__ out, const int* __restrict__ tokens,
    const int* __restrict__ positions, int nq, int hd, int window, int max_spans) {
  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int pos = positions[n];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int spans = min(max_spans, (pos - lo) / kSpan + 1);
  const float* src = part + (static_cast<size_t>(blockIdx.x) * nq + h) * max_spans * (hd + 2);
  __shared__ float scratch[16];
  float mine = -INFINITY;
  for (int s = tid; s < spans; s += kThreads) mine = fmaxf(mine, src[s * (hd + 2) + hd]);
  const float M = block_max(mine, scratch);
  const float m_use = M == -INFINITY ? 0.f : M;
  if (tid < hd) {
    float total = 0.f, l = 0.f;
#pragma unroll 8
    for (int s = 0; s < spans; ++s) {
      const float w = expf(src[s * (hd + 2) + hd] - m_use);
      total = fmaf(src[s * (hd + 2) + tid], w, total);
      l = fmaf(src[s * (hd + 2) + hd + 1], w, l);
    }
    out[(static_cast<size_t>(n) * nq + h) * hd + tid] = from_float<TQ>(l > 0.f ? total / l : 0.f);
  }
}

}  // namespace

extern "C" int pyre_attn_generic_spans(int max_keys) { return max_keys <= kSpan ? 1 : (max_keys + kSpan - 1) / kSpan; }

// `max_keys`: no token of the launch sees more keys than this (the block tables' width in tokens
// will do). `part`: scratch of n * nq * pyre_attn_generic_spans(max_keys) * (hd + 2) floats, needed
// when there is more than one span.
extern "C" int pyre_attn_generic(const void* q, void* out, int q_dt, const void* k_cache,
                                 const void* v_cache, int cache_dt, const int* tokens, const int* positions,
                                 const int* seq_of_token, const int* block_table, int table_stride,
                                 int n, int nq, int nkv, int hd, int page_size, float scale,
                                 int window, int max_keys, float* part, int grouped, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(q_dt) && known_dtype(cache_dt), "attn_generic: unknown dtype");
  PYRE_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attn_generic: %d query heads do not divide over %d kv heads", nq, nkv);
  PYRE_REQUIRE(hd > 0 && hd <= kMaxHead, "attn_generic: head_dim %d is outside 1..%d", hd, kMaxHead);
  PYRE_REQUIRE(page_size > 0 && table_stride > 0, "attn_generic: bad page geometry");
  PYRE_REQUIRE(nq <= 65535, "attn_generic: too many heads");
  PYRE_REQUIRE(max_keys > 0, "attn_generic: max_keys=%d", max_keys);
  if (n <= 0) return 0;
  const int spans = pyre_attn_generic_spans(max_keys);
  PYRE_REQUIRE(spans <= 65535, "attn_generic: %d keys are too many for one launch", max_keys);
  PYRE_REQUIRE(spans == 1 || part, "attn_generic: %d spans of keys need scratch memory", spans);
  float* scratch = spans == 1 ? nullptr : part;
  const bool vec = hd % 4 == 0 && page_size % 4 == 0 && reinterpret_cast<uintptr_t>(k_cache) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(v_cache) % 16 == 0;
  if (grouped && vec && q_dt == kF32 && cache_dt == kF32) {
    // the query heads of a key/value head together: the span's keys and values are read once for all of them
    const int per_kv = (nq / nkv + kGroupHeads - 1) / kGroupHeads;
    PYRE_REQUIRE(nkv * per_kv <= 65535, "attn_generic: too many heads");
    hipLaunchKernelGGL(attn_grouped_f32_kernel, dim3(n, nkv * per_kv, spans), dim3(kThreads), 0, stream,
                       static_cast<const float*>(q), static_cast<const float*>(k_cache),
                       static_cast<const float*>(v_cache), static_cast<float*>(out), tokens, positions, seq_of_token,
                       block_table, table_stride, nq, nkv, hd, page_size, scale, window, scratch);
    if (spans > 1)
      hipLaunchKernelGGL((attn_generic_join_kernel<float>), dim3(n, nq), dim3(kThreads), 0, stream, scratch,
                         static_cast<float*>(out), tokens, positions, nq, hd, window, spans);
    return check_launch("attn_generic");
  }
#define PYRE_LAUNCH_GENERIC(VEC)                                                                          \
  PYRE_DISPATCH(q_dt, TQ, PYRE_DISPATCH(cache_dt, TC,                                                     \
      hipLaunchKernelGGL((attn_generic_kernel<TQ, TC, VEC>), dim3(n, nq, spans), dim3(kThreads), 0, stream, \
                         static_cast<const TQ*>(q), static_cast<const TC*>(k_cache),                      \
                         static_cast<const TC*>(v_cache), static_cast<TQ*>(out), tokens, positions,       \
                         seq_of_token, block_table, table_stride, nq, nkv, hd, page_size, scale,          \
                         window, scratch)))
  if (vec) {
    PYRE_LAUNCH_GENERIC(true);
  } else {
    PYRE_LAUNCH_GENERIC(false);
  }
#undef PYRE_LAUNCH_GENERIC
  if (spans > 1) {
    PYRE_DISPATCH(q_dt, TQ,
        hipLaunchKernelGGL((attn_generic_join_kernel<TQ>), dim3(n, nq), dim3(kThreads), 0, stream, scratch,
                           static_cast<TQ*>(out), tokens, positions, nq, hd, window, spans));
  }
  return check_launch("attn_generic");
}
