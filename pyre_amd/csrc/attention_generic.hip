// Causal (optionally windowed) attention of every token of a step over the paged
// cache, for any head size up to 256, any page size, any grouping of heads and
// either element type; all arithmetic fp32. One block per (token, query head).
//
//   scores[j] = (q . k_j) * scale      for lo <= j <= pos     (pyre/model.py:109)
//   probs     = softmax(scores)                               (pyre/model.py:122)
//   out       = sum_j probs[j] v_j                            (pyre/model.py:123)
//
// `tokens` (or null: all of them) lists the n tokens of the flat batch to attend for.
// A token at position `pos` sees the keys lo..pos of its request, all read from
// the cache (this step's keys were written before the call), so prompt portions
// and single decoded tokens are the same case. lo = max(0, pos - window + 1) for
// a window, else 0. The order of every sum depends on (lo, pos) alone, so the
// result for a position does not depend on how the step was cut or batched.
// This is the 32-bit path's attention and the 16-bit path's fallback; it stands
// where the reference has `forward_paged`'s gather + matmuls (pyre/model.py:274-290)
// and its decode kernel (pyre/kernels/paged_attn.py:26-71).
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

constexpr int kThreads = 256;
constexpr int kChunk = 1024;   // keys whose scores are held in LDS at a time
constexpr int kMaxHead = 256;

template <typename TQ, typename TC>
__global__ __launch_bounds__(kThreads) void attn_generic_kernel(
    const TQ* __restrict__ q, const TC* __restrict__ k_cache, const TC* __restrict__ v_cache,
    TQ* __restrict__ out, const int* __restrict__ tokens, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride, int nq, int nkv,
    int hd, int page_size, float scale, int window) {
  __shared__ float qs[kMaxHead];
  __shared__ float sc[kChunk];
  __shared__ float accs[kThreads];
  __shared__ float scratch[16];

  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (nq / nkv);
  const int pos = positions[n];
  const int* table = block_table + static_cast<size_t>(seq_of_token[n]) * table_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;

  for (int d = tid; d < hd; d += kThreads) qs[d] = to_float(q[(static_cast<size_t>(n) * nq + h) * hd + d]);
  __syncthreads();

  // The second product splits the threads into `groups` sets of hd threads;
  // set g takes the keys g, g + groups, ... of a chunk for output element d.
  const int groups = kThreads / hd;  // >= 1 because hd <= 256
  const int g = tid / hd, d = tid % hd;
  const bool active = g < groups;

  float m = -INFINITY, l = 0.f, acc = 0.f;
  for (int base = lo; base <= pos; base += kChunk) {
    const int cnt = min(kChunk, pos - base + 1);
    float lmax = -INFINITY;
    for (int j = tid; j < cnt; j += kThreads) {
      const int key = base + j;
      const int page = table[key / page_size], off = key % page_size;
      float s = -INFINITY;  // a page that is not there (padding rows of a captured step) hides its keys
      if (page >= 0) {
        const TC* kp = k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + off) * hd;
        s = 0.f;
        for (int e = 0; e < hd; ++e) s = fmaf(qs[e], to_float(kp[e]), s);
        s *= scale;
      }
      sc[j] = s;
      lmax = fmaxf(lmax, s);
    }
    const float m_new = fmaxf(m, block_max(lmax, scratch));
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = expf(m - m_use);  // 0 on the first chunk (m = -inf)
    float lsum = 0.f;
    for (int j = tid; j < cnt; j += kThreads) {
      const float p = expf(sc[j] - m_use);
      sc[j] = p;
      lsum += p;
    }
    l = l * alpha + block_sum(lsum, scratch);  // block_sum's barriers publish sc[]
    if (active) {
      acc *= alpha;
      for (int j = g; j < cnt; j += groups) {
        const int key = base + j;
        const int page = table[key / page_size], off = key % page_size;
        if (page < 0) continue;
        const TC* vp = v_cache + ((static_cast<size_t>(page) * nkv + kvh) * hd + d) * page_size + off;
        acc = fmaf(sc[j], to_float(*vp), acc);
      }
    }
    m = m_new;
    __syncthreads();  // sc[] is rewritten by the next chunk
  }

  accs[tid] = active ? acc : 0.f;
  __syncthreads();
  if (tid < hd) {
    float total = 0.f;
    for (int gg = 0; gg < groups; ++gg) total += accs[gg * hd + tid];
    out[(static_cast<size_t>(n) * nq + h) * hd + tid] = from_float<TQ>(l > 0.f ? total / l : 0.f);
  }
}

}  // namespace

extern "C" int pyre_attn_generic(const void* q, void* out, int q_dt, const void* k_cache,
                                 const void* v_cache, int cache_dt, const int* tokens, const int* positions,
                                 const int* seq_of_token, const int* block_table, int table_stride,
                                 int n, int nq, int nkv, int hd, int page_size, float scale,
                                 int window, hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(q_dt) && known_dtype(cache_dt), "attn_generic: unknown dtype");
  PYRE_REQUIRE(nq > 0 && nkv > 0 && nq % nkv == 0, "attn_generic: %d query heads do not divide over %d kv heads", nq, nkv);
  PYRE_REQUIRE(hd > 0 && hd <= kMaxHead, "attn_generic: head_dim %d is outside 1..%d", hd, kMaxHead);
  PYRE_REQUIRE(page_size > 0 && table_stride > 0, "attn_generic: bad page geometry");
  PYRE_REQUIRE(nq <= 65535, "attn_generic: too many heads");
  if (n <= 0) return 0;
  PYRE_DISPATCH(q_dt, TQ, PYRE_DISPATCH(cache_dt, TC,
      hipLaunchKernelGGL((attn_generic_kernel<TQ, TC>), dim3(n, nq), dim3(kThreads), 0, stream,
                         static_cast<const TQ*>(q), static_cast<const TC*>(k_cache),
                         static_cast<const TC*>(v_cache), static_cast<TQ*>(out), tokens, positions,
                         seq_of_token, block_table, table_stride, nq, nkv, hd, page_size, scale,
                         window)));
  return check_launch("attn_generic");
}
