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
#include <type_traits>

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

// The same for the query heads that share a key/value head, float32 throughout, on the matrix
// cores' float32 instruction 16x16x4: one block per (token, key/value head with up to 16 of its
// query heads, span of keys), so that a span's keys and values are read once for the group and
// not once per head (a decode step's attention is all memory traffic). The instruction's 16
// columns are the query heads; its 16 rows are 16 keys (scores) or 16 elements of the head
// (output). It adds an element's products one after the other with fused multiply-adds, in the
// order of its four lane groups, so every sum here is a chain in a fixed order too: a score over
// the head's elements 0, 4, 8, 12, 1, 5, ... of each run of 16 (a lane holds four consecutive
// elements of its key, one 16-byte load), an output element over the keys of the span in the same
// order within each run of 16 keys, the runs in ascending order. Keys are taken in runs of 16 that
// start at multiples of 16 (inside one page: the page size is a multiple of 16); those of a run
// outside lo..pos get the weight 0, and what they hold is finite (older keys of the request) or zero
// (behind its last key). A wave issues the loads of all its keys and values before it multiplies, so
// the whole span is on its way at once. Head sizes that are multiples of 16 up to 128.
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
constexpr int kSingleHeads = 16;

// ALIGNED: no window, so a span starts at a multiple of 128 and touches eight runs; else nine.
// A block takes `per_block` spans of its token one after the other (grid.z blocks cover them all):
// the keys of the next span are asked for as soon as the scores of the current one are computed,
// its values as soon as the current output is, so that a block always has loads on their way while
// it multiplies. What a span's partial result is does not depend on per_block.
// Every span issues the same loads and the same matrix instructions whatever it holds, so that the
// waits for loads count exactly: a run past the span's end or in a page that is not there (padding
// rows of a captured step) reads a run that is there, or page 0, and is made harmless afterwards
// (its scores are -inf, its values zero).
template <int HT, bool ALIGNED>  // head size / 16
__global__ __launch_bounds__(kThreads) void attn_single_f32_kernel(
    const float* __restrict__ q, const float* __restrict__ k_cache, const float* __restrict__ v_cache,
    float* __restrict__ out, const int* __restrict__ tokens, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride, int nq, int nkv,
    int page_size, float scale, int window, float* __restrict__ part, int spans, int per_block) {
  constexpr int hd = 16 * HT;
  constexpr int kRuns = kSpan / 16 + (ALIGNED ? 0 : 1);
  constexpr int kScoreLd = kRuns * 16 + 4, kQLd = hd + 4;  // rows that start four banks apart
  constexpr int kMyRuns = (kRuns + 3) / 4;         // runs of keys whose scores one wave computes
  constexpr int kMyTiles = (HT + 3) / 4;           // tiles of 16 output elements of one wave
  __shared__ __attribute__((aligned(16))) float sc[kSingleHeads][kScoreLd];
  __shared__ __attribute__((aligned(16))) float qs[kSingleHeads][kQLd];
  __shared__ float ml[kSingleHeads][2];  // maximum and sum of each head's span

  const int n = tokens ? tokens[blockIdx.x] : blockIdx.x, tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same for the whole wave, and known to be
  const int lane = tid & 63, g = lane >> 4, c16 = lane & 15;
  const int n_rep = nq / nkv, per_kv = (n_rep + kSingleHeads - 1) / kSingleHeads;
  const int kvh = blockIdx.y / per_kv, head0 = kvh * n_rep + (blockIdx.y % per_kv) * kSingleHeads;
  const int nheads = min(kSingleHeads, kvh * n_rep + n_rep - head0);
  const int pos = positions[n];
  const int* table = block_table + static_cast<size_t>(seq_of_token[n]) * table_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int span0 = static_cast<int>(blockIdx.z) * per_block;
  const int span_end = min(span0 + per_block, (pos - lo) / kSpan + 1);  // the token's spans end here
  if (span0 >= span_end) return;

  // A span: its keys base..last, in `nruns` runs of 16 from `first` on.
  struct Span { int base, last, first, nruns; };
  auto span_at = [&](int span) {
    Span sp;
    sp.base = lo + span * kSpan;
    sp.last = min(pos, sp.base + kSpan - 1);
    sp.first = sp.base & ~15;
    sp.nruns = (sp.last >> 4) - (sp.base >> 4) + 1;
    return sp;
  };
  // The loads of a span's keys (this wave's runs wave, wave + 4, ...) and values (tiles wave,
  // wave + 4 of the head's elements, every run). All of them are issued before anything waits for one.
  f32x4 kreg[kMyRuns][HT];
  bool kthere[kMyRuns];
  auto ask_keys = [&](const Span& sp) {
#pragma unroll
    for (int i = 0; i < kMyRuns; ++i) {
      const int r = wave + 4 * i, key0 = sp.first + 16 * min(r, sp.nruns - 1);
      const int page = table[key0 / page_size];
      kthere[i] = r < sp.nruns && page >= 0;
      const float* kp = k_cache + ((static_cast<size_t>(max(page, 0)) * nkv + kvh) * page_size + key0 % page_size + c16) * hd + 4 * g;
#pragma unroll
      for (int b = 0; b < HT; ++b) kreg[i][b] = *reinterpret_cast<const f32x4*>(kp + 16 * b);
    }
  };
  f32x4 vreg[kRuns][kMyTiles];
  bool vthere[kRuns];
  auto ask_values = [&](const Span& sp) {
#pragma unroll
    for (int r = 0; r < kRuns; ++r) {
      const int key0 = sp.first + 16 * min(r, sp.nruns - 1);
      const int page = table[key0 / page_size];
      vthere[r] = r < sp.nruns && page >= 0;
      const float* vp = v_cache + ((static_cast<size_t>(max(page, 0)) * nkv + kvh) * hd + c16) * page_size + key0 % page_size + 4 * g;
#pragma unroll
      for (int t = 0; t < kMyTiles; ++t)
        if (HT % 4 == 0 || wave + 4 * t < HT) vreg[r][t] = *reinterpret_cast<const f32x4*>(vp + static_cast<size_t>(16 * (wave + 4 * t)) * page_size);
    }
  };
  Span now = span_at(span0);
  ask_keys(now);
  ask_values(now);
  // the queries of the group's heads, through LDS (rows of heads that are not there: zeros)
  for (int i = tid; i < kSingleHeads * (hd / 4); i += kThreads) {
    const int h = i / (hd / 4), e = 4 * (i % (hd / 4));
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (h < nheads) v = *reinterpret_cast<const f32x4*>(q + (static_cast<size_t>(n) * nq + head0 + h) * hd + e);
    *reinterpret_cast<f32x4*>(&qs[h][e]) = v;
  }
  __syncthreads();

  // One span; `ahead`: another one follows, whose loads are issued on the way.
  auto take = [&](int span, auto ahead) {
    const Span next = span_at(span + (ahead ? 1 : 0));
    // Scores: rows are the run's keys, columns the heads; this lane gets keys 4 g .. 4 g + 3 of the run for head c16.
#pragma unroll
    for (int i = 0; i < kMyRuns; ++i) {
      const int r = wave + 4 * i;
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int b = 0; b < HT; ++b) {
        const f32x4 qv = *reinterpret_cast<const f32x4*>(&qs[c16][16 * b + 4 * g]);  // head c16, this lane group's elements
#pragma unroll
        for (int u = 0; u < 4; ++u) s = __builtin_amdgcn_mfma_f32_16x16x4f32(kreg[i][b][u], qv[u], s, 0, 0, 0);
      }
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int key = now.first + 16 * r + 4 * g + u;
        s[u] = kthere[i] && key >= now.base && key <= now.last ? s[u] * scale : -INFINITY;
      }
      if (r < kRuns) *reinterpret_cast<f32x4*>(&sc[c16][16 * r + 4 * g]) = s;
    }
    if (ahead) ask_keys(next);  // into the registers that the scores have just left
    __syncthreads();

    // Softmax of the span, 16 threads a head: thread t of them takes the keys t, t + 16, ... of the runs.
    {
      const int h = tid >> 4, t = tid & 15;
      float p[kRuns], m = -INFINITY;
#pragma unroll
      for (int j = 0; j < kRuns; ++j) m = fmaxf(m, p[j] = sc[h][t + 16 * j]);
#pragma unroll
      for (int x = 8; x > 0; x >>= 1) m = fmaxf(m, __shfl_xor(m, x, 16));
      const float m_use = m == -INFINITY ? 0.f : m;
      float l = 0.f;
#pragma unroll
      for (int j = 0; j < kRuns; ++j) {
        p[j] = expf(p[j] - m_use);  // 0 for the keys outside the span
        sc[h][t + 16 * j] = p[j];
        l += p[j];
      }
#pragma unroll
      for (int x = 8; x > 0; x >>= 1) l += __shfl_xor(l, x, 16);
      if (t == 0) ml[h][0] = m, ml[h][1] = l;
    }
    __syncthreads();

    // Output: rows are 16 elements of the head, columns the heads; the keys of the span run by run.
    f32x4 acc[kMyTiles];
#pragma unroll
    for (int t = 0; t < kMyTiles; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < kRuns; ++r) {
      const f32x4 p = *reinterpret_cast<const f32x4*>(&sc[c16][16 * r + 4 * g]);
#pragma unroll
      for (int t = 0; t < kMyTiles; ++t) {
        if (HT % 4 != 0 && wave + 4 * t >= HT) continue;
        const f32x4 v = vthere[r] ? vreg[r][t] : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int u = 0; u < 4; ++u) acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(v[u], p[u], acc[t], 0, 0, 0);
      }
    }
    if (ahead) ask_values(next);
    if (c16 < nheads) {
      const int h = head0 + c16;
      const float m = ml[c16][0], l = ml[c16][1];
#pragma unroll
      for (int t = 0; t < kMyTiles; ++t) {
        if (HT % 4 != 0 && wave + 4 * t >= HT) continue;
        const int d = 16 * (wave + 4 * t) + 4 * g;  // this lane's four elements
        if (part) {  // [token of the list][head][span][hd + 2]: unnormalised output, max, sum
          float* dst = part + ((static_cast<size_t>(blockIdx.x) * nq + h) * spans + span) * (hd + 2);
          *reinterpret_cast<f32x2*>(dst + d) = f32x2{acc[t][0], acc[t][1]};  // rows of hd + 2 floats start on 8 bytes
          *reinterpret_cast<f32x2*>(dst + d + 2) = f32x2{acc[t][2], acc[t][3]};
          if (d == 0) dst[hd] = m, dst[hd + 1] = l;
        } else {
          f32x4 o;
#pragma unroll
          for (int u = 0; u < 4; ++u) o[u] = l > 0.f ? acc[t][u] / l : 0.f;
          *reinterpret_cast<f32x4*>(out + (static_cast<size_t>(n) * nq + h) * hd + d) = o;
        }
      }
    }
    now = next;
    if (ahead) __syncthreads();  // the scores and the sums are read; the next span may write them
  };
  int span = span0;
  for (; span + 1 < span_end; ++span) take(span, std::true_type{});
  take(span, std::false_type{});
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
                                 int window, int max_keys, float* part, int matrix_cores, hipStream_t stream) {
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
  const bool aligned = reinterpret_cast<uintptr_t>(q) % 16 == 0 && reinterpret_cast<uintptr_t>(out) % 16 == 0 &&
                       (!scratch || reinterpret_cast<uintptr_t>(scratch) % 8 == 0);
  if (matrix_cores && vec && aligned && q_dt == kF32 && cache_dt == kF32 && hd % 16 == 0 && hd <= 128 && page_size % 16 == 0) {
    // the query heads of a key/value head together: the span's keys and values are read once for all of them
    const int per_kv = (nq / nkv + kSingleHeads - 1) / kSingleHeads;
    PYRE_REQUIRE(nkv * per_kv <= 65535, "attn_generic: too many heads");
    // spans a block: as many as leave two blocks a compute unit (the blocks that fit there at once), up to eight
    int per_block = static_cast<int>(static_cast<long>(n) * nkv * per_kv * spans / (2L * compute_units()));
    per_block = max(1, min(8, per_block));
#define PYRE_SINGLE_AS(HT, ALIGNED)                                                                                  \
  hipLaunchKernelGGL((attn_single_f32_kernel<HT, ALIGNED>), dim3(n, nkv * per_kv, (spans + per_block - 1) / per_block), \
                     dim3(kThreads), 0, stream, static_cast<const float*>(q), static_cast<const float*>(k_cache),     \
                     static_cast<const float*>(v_cache), static_cast<float*>(out), tokens, positions, seq_of_token,   \
                     block_table, table_stride, nq, nkv, page_size, scale, window, scratch, spans, per_block)
#define PYRE_SINGLE(HT)                     \
  case HT:                                  \
    if (window > 0) PYRE_SINGLE_AS(HT, false); \
    else PYRE_SINGLE_AS(HT, true);          \
    break
    switch (hd / 16) {
      PYRE_SINGLE(1); PYRE_SINGLE(2); PYRE_SINGLE(3); PYRE_SINGLE(4); PYRE_SINGLE(5); PYRE_SINGLE(6); PYRE_SINGLE(7); PYRE_SINGLE(8);
    }
#undef PYRE_SINGLE
#undef PYRE_SINGLE_AS
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
