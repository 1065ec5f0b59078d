// bfloat16 attention over the paged cache on the matrix cores (MFMA 16x16x32),
// for head sizes that are multiples of 32 up to 256 and page sizes that are
// multiples of 16. Two kernels share one inner loop on 16x16x32 tiles:
//
//   attn_decode_work_kernel  one new token per request; the keys of a request are
//                        dealt to blocks of four waves by a work list that the host
//                        plans in proportion to the contexts, each wave with a
//                        partial result (max, sum, unnormalised output); the waves
//                        of a block join theirs through LDS, the blocks of a request
//                        through memory in the block that finishes last. One wave
//                        serves up to 16 query heads that share a key/value head, so
//                        K and V are read once per group.
//   attn_prefill_kernel  portions of prompts: a wave takes 32 consecutive tokens
//                        of one request and one query head; the four waves of a
//                        block take four heads of one key/value head, so their
//                        K/V reads hit the same cache lines.
//
// and attn_prefill_tile32_kernel, for heads of up to 128 elements, takes prompt
// portions on 32x32x16 tiles with K and V staged through LDS (see there).
//
// All compute the transposed problem so that no operand needs a transpose:
//   S^T[key, col]  = K[key, :] . Q[col, :]          A = K rows (cache, as stored)
//   O^T[d, col]   += V^T[d, key] P^T[key, col]      A = V^T rows (cache stores V
//                                                       transposed), B = P^T, which
//                                                       is exactly the register
//                                                       layout S^T comes out in.
// A "column" is a query head (decode) or a token (prefill). Scores, softmax and
// the output accumulators are fp32 (pyre/model.py:109-123; the reference's own
// decode kernel is pyre/kernels/paged_attn.py:26-71).
#include <type_traits>

#include "pyre_api.h"
#include "pyre_common.h"
#include "pyre_vec4.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kChunk = 32;  // keys per iteration: two MFMA row tiles

__device__ inline bf16x8 load_b128(const bf16* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
// The same for data that is read once: it is not to displace other lines from the caches.
__device__ inline bf16x8 load_b128_stream(const bf16* p) {
  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  return __builtin_bit_cast(bf16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
__device__ inline bf16x8 zero_b128() {
  uint4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}
__device__ inline uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }

// Addressing of one request's keys and values for one key/value head.
struct KV {
  const bf16* k;     // layer slab [pages, nkv, page_size, HD]
  const bf16* v;     // layer slab [pages, nkv, HD, page_size]
  const int* table;  // the request's block table
  int nkv, kvh, page_size;
};

// Per-column causal window: column c sees keys in [lo[c], hi[c]].
template <int CT>
struct Bounds {
  int lo[CT], hi[CT];
};

// One chunk of 32 keys starting at key0 for CT tiles of 16 columns.
//   q[ct][c]   B operands of Q^T, c = 32-wide slice of the head
//   o[dt][ct]  accumulators of O^T, dt = 16-wide slice of the head
//   m, l       running max (in log2 units) and sum of each lane's column
//   load_k(t, c)  A operand of key tile t (16 keys), head slice c: lane (r, g) gets
//                 K[key0 + 16 t + r][32 c + 8 g .. + 8]
//   load_v(dt)    A operand of V^T rows 16 dt + r: slots 0..3 = keys 4g..4g+3 of
//                 tile 0, slots 4..7 = the same keys of tile 1
//   tile_ok[t]    false for a tile whose page is not there: all its keys are hidden
// `edge` says that some key of the chunk may be hidden from some column;
// interior chunks skip all masking.
// RUNS8 deals the keys to the tiles differently, so that a lane's eight values of P^T
// belong to eight consecutive keys and V^T comes in 16-byte loads: row 4 g + j of tile t
// is key key0 + 8 g + 4 t + j; load_k(t, c) gives lane (r, g) the row of key
// key0 + 8 (r / 4) + 4 t + r % 4, load_v(dt) the keys 8 g .. 8 g + 7 in its slots, and
// tile_ok[h] stands for the chunk's keys 16 h .. 16 h + 15.
template <int HD, int CT, bool RUNS8 = false, typename LoadK, typename LoadV>
__device__ inline void attend_core(int key0, bool edge, const bool (&tile_ok)[2], const Bounds<CT>& bd,
                                   float scale_log2, const bf16x8 (&q)[CT][HD / 32],
                                   f32x4 (&o)[HD / 16][CT], float (&m)[CT], float (&l)[CT],
                                   LoadK&& load_k, LoadV&& load_v) {
  const int g = (threadIdx.x & 63) >> 4;
  // S^T tiles: rows = keys key0 + 16 t + (4 g + j), columns = lane's column r.
  f32x4 s[2][CT];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) s[t][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
    if (!RUNS8 && !tile_ok[t]) continue;
#pragma unroll
    for (int c = 0; c < HD / 32; ++c) {
      const bf16x8 a = load_k(t, c);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        s[t][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, q[ct][c], s[t][ct], 0, 0, 0);
    }
  }

  // Online softmax per column; P^T packed as the B operand of the second product:
  // slots 0..3 of a lane are keys 4g..4g+3 of tile 0, slots 4..7 those of tile 1.
  bf16x8 p[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float x[8];
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float v = s[t][ct][j] * scale_log2;
        if (edge) {
          const int key = key0 + (RUNS8 ? 8 * g + 4 * t + j : 16 * t + 4 * g + j);
          if (!tile_ok[RUNS8 ? g >> 1 : t] || key < bd.lo[ct] || key > bd.hi[ct]) v = -INFINITY;
        }
        x[4 * t + j] = v;
        mx = fmaxf(mx, v);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m[ct], mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // column without a visible key so far
    const float alpha = __builtin_amdgcn_exp2f(m[ct] - m_use);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      x[i] = __builtin_amdgcn_exp2f(x[i] - m_use);
      sum += x[i];
    }
    sum += __shfl_xor(sum, 16, 64);
    sum += __shfl_xor(sum, 32, 64);
    l[ct] = l[ct] * alpha + sum;
    m[ct] = m_new;
    uint4 u = {pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
    p[ct] = __builtin_bit_cast(bf16x8, u);
    // Once the running maxima have settled alpha is exactly 1 in every lane: skip
    // the rescaling of the accumulators then.
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < HD / 16; ++dt) o[dt][ct] *= alpha;
    }
  }

  // O^T += V^T P^T.
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    const bf16x8 a = load_v(dt);
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
      o[dt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p[ct], o[dt][ct], 0, 0, 0);
  }
}

// The chunk's operands straight from the paged cache (no LDS): K rows as stored,
// V^T as two runs of four keys, 8 bytes each in the transposed cache.
template <int HD, int CT>
__device__ inline void attend_chunk(const KV& kv, int key0, bool edge, const Bounds<CT>& bd,
                                    float scale_log2, const bf16x8 (&q)[CT][HD / 32],
                                    f32x4 (&o)[HD / 16][CT], float (&m)[CT], float (&l)[CT]) {
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const bf16* kp[2];
  const bf16* vp[2];
  bool ok[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int k0 = key0 + 16 * t;
    const int page = kv.table[k0 / kv.page_size], off = k0 % kv.page_size;
    ok[t] = page >= 0;  // released or never allocated: every key of it is hidden
    const size_t base = static_cast<size_t>(ok[t] ? page : 0) * kv.nkv + kv.kvh;
    kp[t] = kv.k + (base * kv.page_size + off + r) * HD + 8 * g;
    vp[t] = kv.v + (base * HD + r) * kv.page_size + off + 4 * g;
  }
  attend_core<HD, CT>(
      key0, edge, ok, bd, scale_log2, q, o, m, l,
      [&](int t, int c) { return load_b128(kp[t] + 32 * c); },
      [&](int dt) {
        uint2 h[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          h[t] = uint2{0u, 0u};
          if (ok[t]) h[t] = *reinterpret_cast<const uint2*>(vp[t] + static_cast<size_t>(dt) * 16 * kv.page_size);
        }
        const uint4 u = {h[0].x, h[0].y, h[1].x, h[1].y};
        return __builtin_bit_cast(bf16x8, u);
      });
}

// A chunk's operands held in registers, so that the loads of the next chunk can be
// in flight while the current one is multiplied. Keys are dealt as attend_core's RUNS8
// says: a lane's part of V^T is one 16-byte run of eight keys.
template <int HD>
struct ChunkRegs {
  bf16x8 k[2][HD / 32];
  bf16x8 v[HD / 16];
  bool ok[2];  // the pages of the chunk's keys 0..15 and 16..31 are there
};

// 64 consecutive entries of a request's block table, one in each lane of a wave: a
// chunk's pages then come out of a register, not out of a load that the chunk's own
// loads would have to wait for. Entries are asked for in rising order.
struct TableWindow {
  const int* table;
  int width;  // entries of the request's row
  int first;  // the entry that lane 0 holds
  int held;
  __device__ void fill(int entry) {
    first = entry;
    const int i = entry + static_cast<int>(threadIdx.x & 63);
    held = i < width ? table[i] : -1;
  }
  // `entry` is the same in all lanes.
  __device__ int page(int entry) {
    if (entry - first >= 64) fill(entry);
    return __builtin_amdgcn_readlane(held, entry - first);
  }
};

template <int HD, bool STREAM_V>
__device__ inline void load_chunk(const KV& kv, TableWindow& tw, int key0, ChunkRegs<HD>& cr) {
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  size_t base[2];  // (page, key/value head) of each half, in units of page_size * HD elements
  int off[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int k0 = key0 + 16 * h;
    const int entry = k0 / kv.page_size;
    const int page = tw.page(entry);
    off[h] = k0 - entry * kv.page_size;
    cr.ok[h] = page >= 0;
    base[h] = static_cast<size_t>(cr.ok[h] ? page : 0) * kv.nkv + kv.kvh;
  }
  // K: rows 0..7 of a tile are keys of the first half, rows 8..15 of the second.
  const int kh = r >> 3;
  const bool k_ok = kh ? cr.ok[1] : cr.ok[0];
  const bf16* kp = kv.k + ((kh ? base[1] : base[0]) * kv.page_size + (kh ? off[1] : off[0]) + 8 * ((r >> 2) & 1) + (r & 3)) * HD + 8 * g;
#pragma unroll
  for (int t = 0; t < 2; ++t)
#pragma unroll
    for (int c = 0; c < HD / 32; ++c) cr.k[t][c] = k_ok ? load_b128(kp + 4 * t * HD + 32 * c) : zero_b128();
  // V^T: lanes g = 0, 1 take keys of the first half, g = 2, 3 of the second.
  const int vh = g >> 1;
  const bool v_ok = vh ? cr.ok[1] : cr.ok[0];
  const bf16* vp = kv.v + ((vh ? base[1] : base[0]) * HD + r) * kv.page_size + (vh ? off[1] : off[0]) + 8 * (g & 1);
  // STREAM_V (pages of at most 32 keys): the 16 rows of a load are whole cache lines, and
  // these lines, read once, go past the caches. Halves of lines would come from memory twice.
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) {
    const bf16* p = vp + static_cast<size_t>(dt) * 16 * kv.page_size;
    cr.v[dt] = !v_ok ? zero_b128() : STREAM_V ? load_b128_stream(p) : load_b128(p);
  }
}

template <int HD, int CT>
__device__ inline void attend_regs(const ChunkRegs<HD>& cr, int key0, bool edge, const Bounds<CT>& bd,
                                   float scale_log2, const bf16x8 (&q)[CT][HD / 32],
                                   f32x4 (&o)[HD / 16][CT], float (&m)[CT], float (&l)[CT]) {
  const bool ok[2] = {cr.ok[0], cr.ok[1]};
  attend_core<HD, CT, true>(
      key0, edge, ok, bd, scale_log2, q, o, m, l, [&](int t, int c) { return cr.k[t][c]; },
      [&](int dt) { return cr.v[dt]; });
}

// ---------------------------------------------------------------------------
// Decode: grid (nkv * qtiles, capacity of the work list), 4 waves. The blocks of one row of
// the list (one per key/value head and group of 16 query heads) are neighbours in the order
// of dispatch, so that the list's order, longest first, is the order in which work starts. The host deals the
// keys of every request to blocks in proportion to its context, so that a step whose
// requests differ widely in length keeps all compute units busy for the same time:
//   work[0]     = (blocks in the list, -, -, -, -, -, -, -)
//   work[1 + i] = (token in the flat batch, block b of its request + 65536 * blocks nb of its
//                  request, chunks of 32 keys per wave of this request, first partial slot of
//                  the request, the token's position, its request's row of the block table, -, -)
// Block b takes the chunks first + 4 b per .. of its request, a run of `per` chunks for each
// of its four waves, and joins their results through LDS. A request with one block is
// finished by it. Otherwise each block stores its joined partial result (max, sum,
// unnormalised output) at slot (first slot + b) with stores that go through to memory and
// counts itself in at the request's counter; the block that arrives last reads all nb
// partial results with loads that come from memory and joins them in the order 0..nb-1,
// whichever block it is. It leaves the counter at zero. Blocks past the list's end exit.
// ---------------------------------------------------------------------------
constexpr int kMaxBlocksPerRequest = 64;
typedef unsigned u32x4_t __attribute__((ext_vector_type(4)));

// 16- and 4-byte accesses that go through to memory (buffer instructions with the sc0 and
// sc1 bits): what one block stores this way, a block on another die reads this way, within
// one kernel, once the first has waited for its stores and the second has seen a counter move.
__device__ inline __amdgpu_buffer_rsrc_t rsrc_of(const void* p) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, 0x7fffffff, 0x00020000);
}
constexpr int kThrough = 1 | 16;
__device__ inline void store_through(float* base, int elem, f32x4 v) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4_t, v), rsrc_of(base), 4 * elem, 0, kThrough);
}
__device__ inline void store_through(float* base, int elem, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, v), rsrc_of(base), 4 * elem, 0, kThrough);
}
__device__ inline f32x4 load_through4(const float* base, int elem) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc_of(base), 4 * elem, 0, kThrough));
}
__device__ inline float load_through(const float* base, int elem) {
  return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc_of(base), 4 * elem, 0, kThrough));
}


// A barrier that waits for this wave's LDS traffic only. __syncthreads() also waits for
// every global load in flight, which would put the latency of the next chunks' loads
// into each half-step.
__device__ inline void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// What the kernel needs to finish the step's q/k/v product itself (FUSED): the product's partial
// sums [n_partials][rows][(nq + 2 nkv) HD] float32 with its bias, the rotary tables, and where each
// token's key and value go. Every block sums, biases and rotates the queries of its heads into LDS
// (the arithmetic of rope_kv_write, so the same bits); of the waves that attend for a token and
// key/value head, the one whose chunks hold the token's own position first writes its rotated key
// and its value into the cache, zeroes the values behind it in the page as rope_kv_write does, waits
// for the stores and then loads its chunks: no other wave reads that position. A step of single
// tokens then needs no kernel between the product and the attention.
struct RopeIn {
  const float* qkv;
  int n_partials;
  long partial_stride;
  const void* bias;
  int bias_dt;
  const float* cos_t;
  const float* sin_t;
  const int* slots;  // the cache slot of each token, -1: not stored
  int n_rows;        // tokens in the step (rows of the product)
  int write_kv;      // this layer keeps its keys and values
};

// k_cache and v_cache carry no __restrict__: the FUSED form writes through them what it reads later.
#define PYRE_DECODE_WORK_PARAMS                                                                                   \
  const bf16 *__restrict__ q, bf16 *k_cache, bf16 *v_cache,                                                       \
      const int4 *__restrict__ work, const int *__restrict__ positions, const int *__restrict__ seq_of_token,     \
      const int *__restrict__ block_table, int table_stride, float *__restrict__ part_acc,                        \
      float *__restrict__ part_ml, int *__restrict__ counters, bf16 *__restrict__ out, int nq, int nkv,           \
      int page_size, float scale_log2, int window
#define PYRE_DECODE_WORK_ARGS                                                                                     \
  q, k_cache, v_cache, work, positions, seq_of_token, block_table, table_stride, part_acc, part_ml, counters, out, \
      nq, nkv, page_size, scale_log2, window

template <int HD, bool STREAM_V, bool FUSED>
__device__ __forceinline__ void attn_decode_work_block(PYRE_DECODE_WORK_PARAMS, const RopeIn& rope) {
  const int4 head_of_list = work[0];
  if (static_cast<int>(blockIdx.y) >= head_of_list.x) return;
  const int4 item = work[2 * (1 + blockIdx.y)], place = work[2 * (1 + blockIdx.y) + 1];
  const int tok = item.x, b = item.y & 0xffff, nb = item.y >> 16, per = item.z, slot0 = item.w;
  // a list that does not fit the launch is not followed
  if (nb < 1 || nb > kMaxBlocksPerRequest || b < 0 || b >= nb || slot0 < 0 || slot0 + nb > static_cast<int>(gridDim.y) || per < 1)
    return;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int n_rep = nq / nkv, qtiles = (n_rep + 15) / 16;
  const int kvh = blockIdx.x / qtiles, qt = blockIdx.x % qtiles;
  const int head0 = kvh * n_rep + qt * 16, nheads = min(16, n_rep - qt * 16);
  // the token's position and its request's row of the block table come with the list: nothing else
  // stands between the list and the first loads of keys
  const int pos = place.x;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;

  KV kv{k_cache, v_cache, block_table + static_cast<size_t>(place.y) * table_stride, nkv, kvh, page_size};
  Bounds<1> bd{{lo}, {pos}};

  const int first = lo / kChunk, last = pos / kChunk;
  const int begin = first + (4 * b + wave) * per, end = min(last + 1, begin + per);  // may be empty

  static_assert(!FUSED || HD <= 128, "the form that finishes the product itself: heads of up to 128 elements");
  bf16x8 qr[1][HD / 32];
  if constexpr (!FUSED) {
#pragma unroll
    for (int c = 0; c < HD / 32; ++c)
      qr[0][c] = r < nheads ? load_b128(q + (static_cast<size_t>(tok) * nq + head0 + r) * HD + 32 * c + 8 * g) : zero_b128();
  }
  f32x4 o[HD / 16][1];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) o[dt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m[1] = {-INFINITY}, l[1] = {0.f};
  if constexpr (HD <= 128) {
    // Two register sets: while one chunk is multiplied the next one's loads are in flight; the wave
    // starts with both on their way.
    ChunkRegs<HD> ra, rb;
    // No entry beyond those of the chunks up to `last` is read.
    TableWindow tw{kv.table, min(table_stride, (last * kChunk + 16) / page_size + 1), 0, -1};
    if (begin < end) tw.fill(begin * kChunk / page_size);
    // FUSED: of the waves that attend for a token and key/value head (the first group of query heads
    // only), the one whose chunks hold the token's own position writes its key and value; it loads
    // that chunk only when its stores have arrived.
    const bool may_write = FUSED && qt == 0 && rope.write_kv && begin <= last && last < end;
    bool writes = false;
    auto arrived = [&](int c) {
      if (FUSED && writes && c == last) asm volatile("s_waitcnt vmcnt(0)" : : : "memory");
    };
    const bool ask_a = begin < end && !(may_write && begin == last);
    const bool ask_b = begin + 1 < end && !(may_write && begin + 1 == last);
    if constexpr (FUSED) {
      constexpr int half = HD / 2;
      const int width = (nq + 2 * nkv) * HD;
      const float* row = rope.qkv + static_cast<size_t>(tok) * width;
      auto value4 = [&](int col) {  // the product's sum with its bias, four columns from `col` (a multiple of 4) on
        float4 v = sum_partials4<float>(row + col, static_cast<size_t>(rope.partial_stride), rope.n_partials);
        if (rope.bias)
          v = add4(v, rope.bias_dt == kF32 ? Vec4<float>::load(static_cast<const float*>(rope.bias) + col)
                                           : Vec4<bf16>::load(static_cast<const bf16*>(rope.bias) + col));
        return v;
      };
      // elements j..j+3 and half + j.. of the head at `base`: what is loaded, and the rotation of it
      struct Pairs { float4 x1, x2, c4, s4; };
      auto pairs_of = [&](int base, int j) {
        const size_t t = static_cast<size_t>(pos) * half + j;
        return Pairs{value4(base + j), value4(base + j + half), Vec4<float>::load(rope.cos_t + t), Vec4<float>::load(rope.sin_t + t)};
      };
      auto rotate = [&](const Pairs& p, float4& a4, float4& b4) {
        rotate_pair(p.x1.x, p.x2.x, p.c4.x, p.s4.x, a4.x, b4.x);
        rotate_pair(p.x1.y, p.x2.y, p.c4.y, p.s4.y, a4.y, b4.y);
        rotate_pair(p.x1.z, p.x2.z, p.c4.z, p.s4.z, a4.z, b4.z);
        rotate_pair(p.x1.w, p.x2.w, p.c4.w, p.s4.w, a4.w, b4.w);
      };
      // First everything this thread has to load of the product: four pairs of a query (thread it of the
      // block: head it / (HD / 8)), and in the wave that may write, four pairs of the key (lanes
      // 0 .. HD / 8 - 1) or four elements of the value (the next HD / 4 lanes). Then the chunks' loads, which
      // queue behind them; then the arithmetic of rope_kv_write.
      const int it = threadIdx.x;
      const bool q_item = it < nheads * (HD / 8);
      const bool key_lane = may_write && lane < HD / 8, value_lane = may_write && lane >= HD / 8 && lane < HD / 8 + HD / 4;
      const float4 zero4 = {0.f, 0.f, 0.f, 0.f};
      Pairs qp{zero4, zero4, zero4, zero4}, kp = qp;
      float4 vv = zero4;
      if (q_item) qp = pairs_of((head0 + it / (HD / 8)) * HD, 4 * (it % (HD / 8)));
      if (key_lane) kp = pairs_of((nq + kvh) * HD, 4 * lane);
      if (value_lane) vv = value4((nq + nkv + kvh) * HD + 4 * (lane - HD / 8));
      const int slot = may_write ? rope.slots[tok] : -1;
      if (ask_a) load_chunk<HD, STREAM_V>(kv, tw, begin * kChunk, ra);
      if (ask_b) load_chunk<HD, STREAM_V>(kv, tw, (begin + 1) * kChunk, rb);
      // the queries of this block's heads, rounded to bfloat16 as rope_kv_write stores them
      __shared__ __attribute__((aligned(16))) bf16 q_s[16][HD + 8];
      static_assert(16 * (HD / 8) <= 256, "one item of the queries per thread");
      if (q_item) {
        float4 a4, b4;
        rotate(qp, a4, b4);
        const int h = it / (HD / 8), j = 4 * (it % (HD / 8));
        Vec4<bf16>::store(&q_s[h][j], a4);
        Vec4<bf16>::store(&q_s[h][j + half], b4);
      }
      lds_barrier();  // waits for LDS alone: the chunks' loads stay on their way
#pragma unroll
      for (int c = 0; c < HD / 32; ++c) qr[0][c] = r < nheads ? load_b128(&q_s[r][32 * c + 8 * g]) : zero_b128();
      // the token's own key and value
      writes = may_write && slot >= 0;
      if (writes) {
        const int page = slot / page_size, off = slot % page_size;
        if (key_lane) {
          float4 ka, kb;
          rotate(kp, ka, kb);
          bf16* dst = k_cache + ((static_cast<size_t>(page) * nkv + kvh) * page_size + off) * HD + 4 * lane;
          Vec4<bf16>::store(dst, ka);
          Vec4<bf16>::store(dst + half, kb);
        } else if (value_lane) {
          bf16* vrow = v_cache + ((static_cast<size_t>(page) * nkv + kvh) * HD + 4 * (lane - HD / 8)) * page_size;
          const float vals[4] = {vv.x, vv.y, vv.z, vv.w};
          const bool ends = ends_its_page_run(rope.slots, tok, rope.n_rows, slot, page_size);
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            bf16* one = vrow + u * static_cast<size_t>(page_size);
            one[off] = from_float<bf16>(vals[u]);
            // the step's last token of a page leaves nothing of the page's previous owner behind it
            if (ends) zero_tail(one, off + 1, page_size);
          }
        }
      }
    } else {
      if (ask_a) load_chunk<HD, STREAM_V>(kv, tw, begin * kChunk, ra);
      if (ask_b) load_chunk<HD, STREAM_V>(kv, tw, (begin + 1) * kChunk, rb);
    }
    if (begin < end && !ask_a) {
      arrived(begin);
      load_chunk<HD, STREAM_V>(kv, tw, begin * kChunk, ra);
    }
    if (begin + 1 < end && !ask_b) {
      arrived(begin + 1);
      load_chunk<HD, STREAM_V>(kv, tw, (begin + 1) * kChunk, rb);
    }
    for (int c = begin; c < end; c += 2) {
      attend_regs<HD, 1>(ra, c * kChunk, c == first || c == last, bd, scale_log2, qr, o, m, l);
      if (c + 2 < end) {
        arrived(c + 2);
        load_chunk<HD, STREAM_V>(kv, tw, (c + 2) * kChunk, ra);
      }
      if (c + 1 < end) {
        attend_regs<HD, 1>(rb, (c + 1) * kChunk, c + 1 == first || c + 1 == last, bd, scale_log2, qr, o, m, l);
        if (c + 3 < end) {
          arrived(c + 3);
          load_chunk<HD, STREAM_V>(kv, tw, (c + 3) * kChunk, rb);
        }
      }
    }
  } else {
    for (int c = begin; c < end; ++c)
      attend_chunk<HD, 1>(kv, c * kChunk, c == first || c == last, bd, scale_log2, qr, o, m, l);
  }

  // The block's four waves: sum_w o_w 2^(m_w - M), sum_w l_w 2^(m_w - M), M = max_w m_w, waves in the order 0..3.
  __shared__ float acc_s[4][16][HD + 4];
  __shared__ float ml_s[4][16][2];
  if (g == 0) {
    ml_s[wave][r][0] = m[0];
    ml_s[wave][r][1] = l[0];
  }
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt) *reinterpret_cast<f32x4*>(&acc_s[wave][r][dt * 16 + 4 * g]) = o[dt][0];
  __syncthreads();
  const int n_items = gridDim.x;
  float* pa = part_acc + (static_cast<size_t>(slot0 + b) * n_items + blockIdx.x) * 16 * HD;
  float* pm = part_ml + (static_cast<size_t>(slot0 + b) * n_items + blockIdx.x) * 32;
  for (int i = threadIdx.x; i < nheads * (HD / 4); i += 256) {
    const int h = i / (HD / 4), d = 4 * (i % (HD / 4));
    float M = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) M = fmaxf(M, ml_s[w][h][0]);
    float L = 0.f;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = ml_s[w][h][0];
      const float ww = mw == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mw - M);
      L += ml_s[w][h][1] * ww;
      sum += *reinterpret_cast<const f32x4*>(&acc_s[w][h][d]) * ww;
    }
    if (nb == 1) {
      // L is 0 only for a row that sees no key at all (padding of a captured step).
      const float inv = L > 0.f ? 1.f / L : 0.f;
      *reinterpret_cast<uint2*>(out + (static_cast<size_t>(tok) * nq + head0 + h) * HD + d) =
          uint2{pack2(sum[0] * inv, sum[1] * inv), pack2(sum[2] * inv, sum[3] * inv)};
    } else {
      store_through(pa, h * HD + d, sum);
      if (d == 0) {
        store_through(pm, 2 * h, M);
        store_through(pm, 2 * h + 1, L);
      }
    }
  }
  if (nb == 1) return;

  // Count this block in once all its stores have arrived; the last one joins the request's blocks.
  __shared__ int last_s;
  __shared__ float ml_all[kMaxBlocksPerRequest][16][2];
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  if (threadIdx.x == 0) {
    int* counter = counters + static_cast<size_t>(slot0) * n_items + blockIdx.x;
    const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_s = before == nb - 1;
    if (last_s) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!last_s) return;
  const float* pa0 = part_acc + (static_cast<size_t>(slot0) * n_items + blockIdx.x) * 16 * HD;
  const float* pm0 = part_ml + (static_cast<size_t>(slot0) * n_items + blockIdx.x) * 32;
  const int acc_step = n_items * 16 * HD, ml_step = n_items * 32;  // floats from one block's slot to the next
  for (int i = threadIdx.x; i < nb * 32; i += 256) {
    const int bb = i >> 5, j = i & 31;
    ml_all[bb][j >> 1][j & 1] = load_through(pm0 + static_cast<size_t>(bb) * ml_step, j);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < nheads * (HD / 4); i += 256) {
    const int h = i / (HD / 4), d = 4 * (i % (HD / 4));
    float M = -INFINITY;
    for (int bb = 0; bb < nb; ++bb) M = fmaxf(M, ml_all[bb][h][0]);
    float L = 0.f;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    constexpr int kAtOnce = 8;  // loads in flight
    for (int b0 = 0; b0 < nb; b0 += kAtOnce) {
      f32x4 v[kAtOnce];
#pragma unroll
      for (int u = 0; u < kAtOnce; ++u)
        if (b0 + u < nb) v[u] = load_through4(pa0 + static_cast<size_t>(b0 + u) * acc_step, h * HD + d);
#pragma unroll
      for (int u = 0; u < kAtOnce; ++u)
        if (b0 + u < nb) {
          const float mb = ml_all[b0 + u][h][0];
          const float wb = mb == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(mb - M);
          L += ml_all[b0 + u][h][1] * wb;
          sum += v[u] * wb;
        }
    }
    const float inv = L > 0.f ? 1.f / L : 0.f;
    *reinterpret_cast<uint2*>(out + (static_cast<size_t>(tok) * nq + head0 + h) * HD + d) =
        uint2{pack2(sum[0] * inv, sum[1] * inv), pack2(sum[2] * inv, sum[3] * inv)};
  }
}

// Two forms of the kernel. The registers of a wave (two chunks of keys and values in flight)
// leave room for two waves per SIMD. When the step has so few requests that a block per
// compute unit covers them, a second block on the same unit would leave another unit idle
// (the dispatcher fills units in order): that form keeps a unit to one block. With more
// requests than units, two blocks per unit hide each other's latencies at start and end.
template <int HD, bool STREAM_V>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_decode_work_alone_kernel(
    PYRE_DECODE_WORK_PARAMS) {
  attn_decode_work_block<HD, STREAM_V, false>(PYRE_DECODE_WORK_ARGS, RopeIn{});
}
template <int HD, bool STREAM_V>
__global__ __launch_bounds__(256, 2) void attn_decode_work_kernel(PYRE_DECODE_WORK_PARAMS) {
  attn_decode_work_block<HD, STREAM_V, false>(PYRE_DECODE_WORK_ARGS, RopeIn{});
}
// The same two forms, finishing the q/k/v product themselves (heads of up to 128 elements).
template <int HD, bool STREAM_V>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_decode_work_rope_alone_kernel(
    PYRE_DECODE_WORK_PARAMS, RopeIn rope) {
  attn_decode_work_block<HD, STREAM_V, true>(PYRE_DECODE_WORK_ARGS, rope);
}
template <int HD, bool STREAM_V>
__global__ __launch_bounds__(256, 2) void attn_decode_work_rope_kernel(PYRE_DECODE_WORK_PARAMS, RopeIn rope) {
  attn_decode_work_block<HD, STREAM_V, true>(PYRE_DECODE_WORK_ARGS, rope);
}
#undef PYRE_DECODE_WORK_PARAMS
#undef PYRE_DECODE_WORK_ARGS

// ---------------------------------------------------------------------------
// Prefill: grid (tiles, nkv * head groups); wave w takes head group*4 + w.
// tiles[i] = (first token of the tile in the flat batch, number of tokens <= 32).
// ---------------------------------------------------------------------------
template <int HD>
__global__ __launch_bounds__(256) void attn_prefill_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ out, const int* __restrict__ tiles, const int* __restrict__ positions,
    const int* __restrict__ seq_of_token, const int* __restrict__ block_table, int table_stride,
    int nq, int nkv, int page_size, float scale_log2, int window) {
  constexpr int CT = 2;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int n_rep = nq / nkv, hgroups = (n_rep + 3) / 4;
  const int kvh = blockIdx.y / hgroups, hg = blockIdx.y % hgroups;
  const int hin = hg * 4 + wave;
  if (hin >= n_rep) return;
  const int head = kvh * n_rep + hin;
  const int t0 = tiles[2 * blockIdx.x], ntok = tiles[2 * blockIdx.x + 1];
  const int pos0 = positions[t0];

  KV kv{k_cache, v_cache, block_table + static_cast<size_t>(seq_of_token[t0]) * table_stride, nkv, kvh, page_size};
  Bounds<CT> bd;
  bf16x8 qr[CT][HD / 32];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = 16 * ct + r;
    const bool live = col < ntok;
    // A column past the tile's end computes on zeros over the first column's keys
    // and is not stored.
    bd.hi[ct] = live ? pos0 + col : pos0;
    bd.lo[ct] = window > 0 ? max(0, bd.hi[ct] - window + 1) : 0;
#pragma unroll
    for (int c = 0; c < HD / 32; ++c)
      qr[ct][c] = live ? load_b128(q + (static_cast<size_t>(t0 + col) * nq + head) * HD + 32 * c + 8 * g) : zero_b128();
  }
  f32x4 o[HD / 16][CT];
#pragma unroll
  for (int dt = 0; dt < HD / 16; ++dt)
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) o[dt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m[CT], l[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) { m[ct] = -INFINITY; l[ct] = 0.f; }

  const int lo_all = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int hi_all = pos0 + ntok - 1;
  const int first = lo_all / kChunk, last = hi_all / kChunk;
  // A chunk is interior when every key of it is visible to every column: it ends
  // at or before the first token's position and starts at or after the highest
  // lower bound of the tile.
  const int lo_max = window > 0 ? max(0, hi_all - window + 1) : 0;
  for (int c = first; c <= last; ++c) {
    const int key0 = c * kChunk;
    const bool edge = key0 + kChunk - 1 > pos0 || key0 < lo_max;
    attend_chunk<HD, CT>(kv, key0, edge, bd, scale_log2, qr, o, m, l);
  }

#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int col = 16 * ct + r;
    if (col >= ntok) continue;
    const float inv = 1.f / l[ct];
    bf16* dst = out + (static_cast<size_t>(t0 + col) * nq + head) * HD + 4 * g;
#pragma unroll
    for (int dt = 0; dt < HD / 16; ++dt) {
      const f32x4 v = o[dt][ct];
      *reinterpret_cast<uint2*>(dst + dt * 16) = uint2{pack2(v[0] * inv, v[1] * inv), pack2(v[2] * inv, v[3] * inv)};
    }
  }
}

// ---------------------------------------------------------------------------
// Prefill on 32x32x16 tiles: the NW waves of a block take NW query heads of one
// key/value head over the same 32 tokens (one MFMA tile of columns per wave);
// keys and values come through LDS in chunks of 64, four stages, loaded once
// per block. Per chunk and wave: S^T (64 keys x 32 tokens) in two tiles, one
// exchange between the two lanes that share a column for the running maximum,
// and O^T (HD x 32) += V^T P^T. The sum of a column is kept per lane (each lane
// adds the keys it holds) and joined once at the end.
//
// The chunks go from the cache straight into LDS (global_load_lds_dwordx4: 16 bytes
// per lane, the 64 pieces of an instruction at consecutive LDS addresses, each from
// an address of its lane's choosing), no register in between: two chunks are in
// flight while two are being read, which hides the latency of L2 and memory that one
// register set per wave could not (a 2,048-token portion after 30,000 tokens took
// 1,230 us per layer on the 7B heads with staging through registers, 900 us with
// loads that always hit). Such loads cannot pad rows, so rows are rotated instead:
//   K    rows of SEGP slots of 16 bytes (SEGP = 4, 8 or 16 >= HD / 8), 64 of them; piece p
//        of row j lies in slot (p + j / RPB) % SEGP, RPB = rows per 256 bytes, so that 16
//        lanes reading the same piece of 16 consecutive rows hit distinct banks.
//        Row 16 h + 8 a + 4 c + b of a tile of 32 holds key 16 h + 8 c + 4 a + b: with the
//        rows in this order the eight scores that a lane packs for one MFMA of the second
//        product belong to eight consecutive keys, and V^T needs no reordering.
//   V^T  four runs of 16 keys, each [HD][16 keys] (32 bytes a row, two pieces); the piece
//        of keys 8 x .. 8 x + 7 of row d lies in slot x ^ ((d >> 3) & 1).
// A page that is not there (released, or past the request's end) is read from 16 bytes of
// zeros instead: all its keys are out of every column's bounds, and a hidden key's value is
// weighted with an exact 0, which only a finite value survives. The slots of a request's last
// page after its last key are finite because they are zero: whoever writes a token into a page
// zeroes the values behind it (pyre_common.h: ends_its_page_run, zero_tail).
// ---------------------------------------------------------------------------
typedef __attribute__((ext_vector_type(16))) float f32x16;
constexpr int kKeys = 64;


// 16 bytes per lane from global memory straight into LDS: lane x's piece lands at
// lds_addr + 16 x. The compiler does not know of these loads; whoever reads the bytes
// waits for them with wait_loads (they finish in the order of issue) and a barrier.
__device__ inline void load_to_lds(const void* src, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory", "m0");
}
template <int N>
__device__ inline void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __attribute__((aligned(16))) const unsigned kZeroPiece[4] = {0u, 0u, 0u, 0u};

//
// work[2 i], work[2 i + 1] = (first token of the tile in the flat batch, tokens <= 32, first
// chunk of 64 keys, last chunk), (first partial slot of the tile, this block's number b among
// the tile's blocks, their number nb, -): the host deals the chunks of a tile to nb blocks
// when there are fewer tiles than compute units (a portion of a prompt late in a long
// context) or when the tiles differ much in length (the triangle of a whole prompt). A tile
// with one block is finished by it. Otherwise every wave stores its head's partial result
// (max, sum, unnormalised output) at slot (first slot + b) with stores that go through to
// memory and counts itself in at the counter of (tile, head); the wave that arrives last
// reads the nb partial results with loads that come from memory and joins them in the order
// 0..nb-1, whichever wave it is, and leaves the counter at zero.
template <int HD, int NW>
__global__ __launch_bounds__(NW * 64) void attn_prefill_tile32_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ v_cache,
    bf16* __restrict__ out, const int4* __restrict__ work, float* __restrict__ partials, int* __restrict__ counters,
    int n_slots, const int* __restrict__ positions, const int* __restrict__ seq_of_token,
    const int* __restrict__ block_table, int table_stride, int nq, int nkv, int page_size, float scale_log2,
    int window) {
  constexpr int SEG = HD / 8;                              // 16-byte pieces of one K row
  constexpr int SEGP = SEG <= 4 ? 4 : SEG <= 8 ? 8 : 16;   // slots of a K row in LDS
  constexpr int KROW = 16 * SEGP;                          // bytes of a K row in LDS
  constexpr int RPB = 16 / SEGP;                           // K rows per 256 bytes
  constexpr int kBytesK = kKeys * KROW, kBytesV = 2 * HD * kKeys, kStage = kBytesK + kBytesV;
  constexpr int VRUN = 32 * HD;                            // bytes of one run of V^T: [HD][16 keys]
  constexpr int NS = 4;                                    // stages: two chunks being read, two in flight
  constexpr int NI = 4;                                    // waves that issue loads: the first wave of each SIMD
  constexpr int KI = kBytesK / 1024, VI = kBytesV / 1024;  // load instructions (1 KB each) per chunk
  constexpr int PER = (KI + VI) / NI;                      // per issuing wave
  static_assert((KI + VI) % NI == 0 && VRUN % 1024 == 0 && NS * kStage <= 160 * 1024 - 1024, "stage geometry");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[NS * kStage];

  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid >> 6), lane = tid & 63, r = lane & 31,
            g = lane >> 5;
  const int n_rep = nq / nkv, hgroups = (n_rep + NW - 1) / NW;
  const int kvh = blockIdx.x / hgroups, hg = blockIdx.x % hgroups;
  const int hin = hg * NW + wave;
  const bool active = hin < n_rep;  // a wave without a head still helps loading
  const int head = kvh * n_rep + (active ? hin : 0);
  const int4 item = work[2 * blockIdx.y], share = work[2 * blockIdx.y + 1];
  const int t0 = item.x, ntok = item.y;
  const int pos0 = positions[t0];
  const int* table = block_table + static_cast<size_t>(seq_of_token[t0]) * table_stride;

  // Column r of this wave: token t0 + r; it sees keys lo..hi.
  const bool live = active && r < ntok;
  const int hi = r < ntok ? pos0 + r : pos0;
  const int lo = window > 0 ? max(0, hi - window + 1) : 0;
  bf16x8 qr[HD / 16];
#pragma unroll
  for (int c = 0; c < HD / 16; ++c)
    qr[c] = live ? load_b128(q + (static_cast<size_t>(t0 + r) * nq + head) * HD + 16 * c + 8 * g) : zero_b128();
  f32x16 o[HD / 32];
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
  float m = -INFINITY, l = 0.f;  // m in raw score units; l is this lane's share of the column's sum

  const int lo_all = window > 0 ? max(0, pos0 - window + 1) : 0;
  const int hi_all = pos0 + ntok - 1;
  // this block's chunks, kept within the tile's whatever the list says
  const int first = min(max(item.z, lo_all / kKeys), hi_all / kKeys), last = min(max(item.w, first), hi_all / kKeys);
  const int lo_max = window > 0 ? max(0, hi_all - window + 1) : 0;

  const int n = last - first + 1;

  // Loads: the first NI waves issue them, instructions wave, wave + NI, ... of the chunk's
  // KI + VI. An instruction's 64 pieces come from one run of 16 keys, so from one page. What
  // is fixed for the whole kernel is worked out here:
  //   global: cache + ((page * nkv + kvh) * page_size * HD + slot * g_mul) + g_lane
  //   LDS:    stage * kStage + g_lds
  const bool issuer = wave < NI;
  const unsigned lds_base = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds)));
  const bf16* g_ptr[PER];
  int g_run[PER], g_mul[PER], g_lane[PER], g_lds[PER];
#pragma unroll
  for (int t = 0; t < PER; ++t) {
    const int j = min(wave, NI - 1) + NI * t;
    g_lds[t] = 1024 * j;
    if (j < KI) {
      const int row = j * (1024 / KROW) + lane / SEGP, slot = lane % SEGP;
      int piece = (slot + SEGP - (row / RPB) % SEGP) % SEGP;
      if (piece >= SEG) piece = 0;  // a slot that no piece maps to (heads of 96): any bytes that are there
      const int in_tile = row & 31;
      const int key = (row & 32) + (in_tile & 16) + 8 * ((in_tile >> 2) & 1) + 4 * ((in_tile >> 3) & 1) + (in_tile & 3);
      g_ptr[t] = k_cache;
      g_run[t] = __builtin_amdgcn_readfirstlane(key >> 4);
      g_mul[t] = HD;
      g_lane[t] = (key & 15) * HD + 8 * piece;
    } else {
      const int jv = j - KI;
      const int d = 32 * (jv % (VRUN / 1024)) + (lane >> 1), half = (lane & 1) ^ ((d >> 3) & 1);
      g_ptr[t] = v_cache;
      g_run[t] = jv / (VRUN / 1024);
      g_mul[t] = 1;
      g_lane[t] = d * page_size + 8 * half;
    }
  }
  // (pi, sl): index into the block table and slot within that page of the first key of
  // the next chunk to look up; both advance by whole runs, without a division per chunk.
  // The pages of a chunk are looked up one chunk ahead of its loads, so that the latency
  // of the table is never waited for.
  int pi = (first * kKeys) / page_size, sl = (first * kKeys) % page_size;
  int run_page[kKeys / 16], run_slot[kKeys / 16];
  auto lookup = [&]() {
#pragma unroll
    for (int run = 0; run < kKeys / 16; ++run) {
      run_page[run] = table[min(pi, table_stride - 1)];
      run_slot[run] = sl;
      sl += 16;
      const bool wrap = sl >= page_size;
      sl = wrap ? 0 : sl;
      pi += wrap ? 1 : 0;
    }
  };
  const size_t page_elems = static_cast<size_t>(page_size) * HD;
  // The chunk whose pages were looked up last goes into `stage`.
  auto issue = [&](int stage) {
    size_t base[kKeys / 16];
    int slot[kKeys / 16];
    bool there[kKeys / 16];
#pragma unroll
    for (int run = 0; run < kKeys / 16; ++run) {
      base[run] = (static_cast<size_t>(max(run_page[run], 0)) * nkv + kvh) * page_elems;
      slot[run] = run_slot[run];
      there[run] = run_page[run] >= 0;
    }
    lookup();  // for the chunk after this one
    const unsigned dst = lds_base + stage * kStage;
#pragma unroll
    for (int t = 0; t < PER; ++t) {
      const int run = g_run[t];
      const size_t b = run == 0 ? base[0] : run == 1 ? base[1] : run == 2 ? base[2] : base[3];
      const int sr = run == 0 ? slot[0] : run == 1 ? slot[1] : run == 2 ? slot[2] : slot[3];
      const bool ok = run == 0 ? there[0] : run == 1 ? there[1] : run == 2 ? there[2] : there[3];
      const bf16* src = ok ? g_ptr[t] + b + sr * g_mul[t] + g_lane[t] : reinterpret_cast<const bf16*>(kZeroPiece);
      load_to_lds(src, dst + g_lds[t]);
    }
  };

  // The loop runs in half-steps with a barrier after each. A wave alternates between a
  // matrix half-step (O^T += V^T P^T of the previous chunk, then S^T of the next) and an
  // arithmetic half-step (softmax of that S^T; the issuing waves ask for the chunk after
  // the next first and wait for the next one last). The second wave of each SIMD
  // (waves NW/2 ..) runs one half-step behind the first, so that at any time one of the
  // two is on the matrix cores and the other on the vector ALU.
  //   chunk x (counted from `first`) is read in half-steps 2x-1 .. 2x+2 and lies in stage
  //   x % 4; its loads are issued in half-step 2x-4, when chunk x-4 was last read in 2x-6,
  //   and have arrived before the barrier that ends half-step 2x-2.
  const int off = NW == 8 ? wave >> 2 : 0;
  if (issuer) {
    lookup();
    issue(0);
  }
  // The query operands have arrived before the loop starts. Without this the compiler,
  // which cannot tell the first round from the others, waits in every round for all loads
  // in flight; here that wait takes in the first chunk, which is needed now anyway.
#pragma unroll
  for (int c = 0; c < HD / 16; ++c) asm volatile("" : "+v"(qr[c]));
  if (issuer) {
    wait_loads<0>();
    if (1 < n) issue(1);
  }
  lds_barrier();
  f32x16 s[2];
  bf16x8 p[2][2];
  const int k_swz = (r / RPB) % SEGP;  // the rotation of row 32 kt + r is the same for both tiles: 32 / RPB is a multiple of SEGP

  // S^T of the chunk in stage sk: tile kt, row i of a lane = key key0 + 32 kt + 16 (i / 8) + 8 g + 4 (i / 4 % 2) + i % 4, column r.
  auto scores = [&](int sk) {
    constexpr int AHEAD = 4;  // head slices whose operands are in flight
    bf16x8 a[AHEAD][2];
    auto load_k = [&](int slot, int cc) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
        a[slot][kt] = *reinterpret_cast<const bf16x8*>(lds + sk * kStage + (32 * kt + r) * KROW + 16 * ((2 * cc + g + k_swz) % SEGP));
    };
#pragma unroll
    for (int cc = 0; cc < AHEAD && cc < HD / 16; ++cc) load_k(cc, cc);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) s[kt][i] = 0.f;
#pragma unroll
    for (int cc = 0; cc < HD / 16; ++cc) {
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
        s[kt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[cc % AHEAD][kt], qr[cc], s[kt], 0, 0, 0);
      if (cc + AHEAD < HD / 16) load_k(cc % AHEAD, cc + AHEAD);
    }
  };
  // O^T += V^T P^T for the chunk in stage sv; MFMA `pair` takes keys 16 pair .. 16 pair + 15, eight per half-wave.
  auto weighted_values = [&](int sv) {
    bf16x8 va[2][HD / 32];
    const int v_lane = r * 32 + 16 * (g ^ ((r >> 3) & 1));
    auto load_v = [&](int slot, int pair) {
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
        va[slot][dt] = *reinterpret_cast<const bf16x8*>(lds + sv * kStage + kBytesK + pair * VRUN + dt * 1024 + v_lane);
    };
    load_v(0, 0);
    load_v(1, 1);
#pragma unroll
    for (int pair = 0; pair < 4; ++pair) {
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
        o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[pair & 1][dt], p[pair >> 1][pair & 1], o[dt], 0, 0, 0);
      if (pair + 2 < 4) load_v(pair & 1, pair + 2);
    }
  };
  // P^T = exp2(S^T scale - running maximum), packed as the next product's operands.
  auto softmax = [&](int key0) {
    if (key0 + kKeys - 1 > pos0 || key0 < lo_max) {  // some key of the chunk may be hidden from some column
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = key0 + 32 * kt + 16 * (i >> 3) + 8 * g + 4 * ((i >> 2) & 1) + (i & 3);
          if (key < lo || key > hi) s[kt][i] = -INFINITY;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int i = 0; i < 16; ++i) mx = fmaxf(mx, s[kt][i]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;  // column without a visible key so far
    const float alpha = __builtin_amdgcn_exp2f((m - m_use) * scale_log2);
    const float mc = m_use * scale_log2;
    m = m_new;
    float sum = 0.f;
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        float x[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          x[e] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][8 * h + e], scale_log2, -mc));
          sum += x[e];
        }
        const uint4 w = {pack2(x[0], x[1]), pack2(x[2], x[3]), pack2(x[4], x[5]), pack2(x[6], x[7])};
        p[kt][h] = __builtin_bit_cast(bf16x8, w);
      }
    l = l * alpha + sum;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) o[dt][i] *= alpha;
    }
  };

  if (off) lds_barrier();  // the second waves start one half-step later
  if (active) scores(0);
  int st = 0;  // stage of chunk c
  for (int c = 0; c < n; ++c) {
    lds_barrier();
    if (issuer && c + 2 < n) issue((st + 2) % NS);
    if (active) softmax((first + c) * kKeys);
    if (issuer) {  // chunk c + 1 is there
      if (c + 2 < n) wait_loads<PER>();
      else wait_loads<0>();
    }
    lds_barrier();
    const int nx = (st + 1) % NS;
    if (active) {
      weighted_values(st);
      if (c + 1 < n) scores(nx);
    }
    st = nx;
  }
  lds_barrier();
  if (!off) lds_barrier();  // every wave passes the same number of barriers

  if (!active) return;
  l += __shfl_xor(l, 32, 64);
  const int slot0 = share.x, b = share.y, nb = share.z;
  if (nb > 1) {
    if (slot0 < 0 || b < 0 || b >= nb || slot0 + nb > n_slots) return;  // a list that does not fit the scratch is not followed
    // floats of one wave's partial result: element (dt, 4 q .. 4 q + 3) of lane x at 4 ((4 dt + q) 64 + x), then (m, l)
    constexpr int kPart = (HD / 32) * 16 * 64 + 2 * 64;
    const size_t per_slot = static_cast<size_t>(gridDim.x) * NW * kPart;
    float* mine = partials + (static_cast<size_t>(slot0 + b) * gridDim.x + blockIdx.x) * NW * kPart + wave * kPart;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int qd = 0; qd < 4; ++qd)
        store_through(mine, 4 * ((4 * dt + qd) * 64 + lane),
                      f32x4{o[dt][4 * qd], o[dt][4 * qd + 1], o[dt][4 * qd + 2], o[dt][4 * qd + 3]});
    store_through(mine, (HD / 32) * 16 * 64 + 2 * lane, m);
    store_through(mine, (HD / 32) * 16 * 64 + 2 * lane + 1, l);
    __builtin_amdgcn_s_waitcnt(0);  // the stores have arrived
    int is_last = 0;
    if (lane == 0) {
      int* counter = counters + (static_cast<size_t>(slot0) * gridDim.x + blockIdx.x) * NW + wave;
      const int before = __hip_atomic_fetch_add(counter, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      is_last = before == nb - 1;
      if (is_last) __hip_atomic_store(counter, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (!__builtin_amdgcn_readfirstlane(is_last)) return;
    const float* theirs = partials + (static_cast<size_t>(slot0) * gridDim.x + blockIdx.x) * NW * kPart + wave * kPart;
    m = -INFINITY;
    l = 0.f;
#pragma unroll
    for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) o[dt][i] = 0.f;
    for (int p = 0; p < nb; ++p, theirs += per_slot) {
      f32x4 v[HD / 32][4];
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd) v[dt][qd] = load_through4(theirs, 4 * ((4 * dt + qd) * 64 + lane));
      const float mp = load_through(theirs, (HD / 32) * 16 * 64 + 2 * lane);
      const float lp = load_through(theirs, (HD / 32) * 16 * 64 + 2 * lane + 1);
      const float m_new = fmaxf(m, mp);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float wa = __builtin_amdgcn_exp2f((m - m_use) * scale_log2);   // 0 for m = -inf
      const float wp = __builtin_amdgcn_exp2f((mp - m_use) * scale_log2);
      m = m_new;
      l = l * wa + lp * wp;
#pragma unroll
      for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
        for (int qd = 0; qd < 4; ++qd)
#pragma unroll
          for (int e = 0; e < 4; ++e) o[dt][4 * qd + e] = o[dt][4 * qd + e] * wa + v[dt][qd][e] * wp;
    }
  }
  if (r >= ntok) return;
  const float inv = 1.f / l;
  bf16* dst = out + (static_cast<size_t>(t0 + r) * nq + head) * HD + 4 * g;
#pragma unroll
  for (int dt = 0; dt < HD / 32; ++dt)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const float v0 = o[dt][4 * b] * inv, v1 = o[dt][4 * b + 1] * inv, v2 = o[dt][4 * b + 2] * inv,
                  v3 = o[dt][4 * b + 3] * inv;
      *reinterpret_cast<uint2*>(dst + 32 * dt + 8 * b) = uint2{pack2(v0, v1), pack2(v2, v3)};
    }
}

template <typename F>
int dispatch_head(int hd, F&& f) {
  switch (hd) {
    case 32: f(std::integral_constant<int, 32>()); return 0;
    case 64: f(std::integral_constant<int, 64>()); return 0;
    case 96: f(std::integral_constant<int, 96>()); return 0;
    case 128: f(std::integral_constant<int, 128>()); return 0;
    case 160: f(std::integral_constant<int, 160>()); return 0;
    case 192: f(std::integral_constant<int, 192>()); return 0;
    case 224: f(std::integral_constant<int, 224>()); return 0;
    case 256: f(std::integral_constant<int, 256>()); return 0;
  }
  return 1;
}

}  // namespace

extern "C" int pyre_attn_mfma_supports(int hd, int page_size, int nq, int nkv) {
  return hd >= 32 && hd <= 256 && hd % 32 == 0 && page_size > 0 && page_size % 16 == 0 && nkv > 0 &&
         nq % nkv == 0;
}

namespace {

int launch_decode_work(const void* q, void* out, void* k_cache, void* v_cache, const int* work, int capacity,
                       const int* positions, const int* seq_of_token, const int* block_table, int table_stride,
                       float* part_acc, float* part_ml, int* counters, int alone, int nq, int nkv, int hd,
                       int page_size, float scale, int window, const RopeIn* rope, hipStream_t stream) {
  PYRE_REQUIRE(pyre_attn_mfma_supports(hd, page_size, nq, nkv),
               "attn_decode_work_bf16: head_dim %d (multiples of 32 up to 256), page_size %d (multiples of 16), "
               "heads %d/%d are not supported", hd, page_size, nq, nkv);
  PYRE_REQUIRE(table_stride > 0 && capacity >= 0, "attn_decode_work_bf16: bad table or capacity");
  PYRE_REQUIRE(reinterpret_cast<uintptr_t>(work) % 16 == 0, "attn_decode_work_bf16: the work list must lie on 16 bytes");  // rows of 8 ints
  if (capacity == 0) return 0;
  const int n_rep = nq / nkv, qtiles = (n_rep + 15) / 16;
  PYRE_REQUIRE(capacity <= 65535, "attn_decode_work_bf16: a list of %d blocks is too long for one launch", capacity);
  const dim3 grid(nkv * qtiles, capacity);
  const float scale_log2 = scale * kLog2e;
#define PYRE_DECODE_LAUNCH_ARGS                                                                                    \
  static_cast<const bf16*>(q), static_cast<bf16*>(k_cache), static_cast<bf16*>(v_cache),                          \
      reinterpret_cast<const int4*>(work), positions, seq_of_token, block_table, table_stride, part_acc, part_ml, \
      counters, static_cast<bf16*>(out), nq, nkv, page_size, scale_log2, window
  const int rc = dispatch_head(hd, [&](auto HDc) {
    constexpr int HD = decltype(HDc)::value;
    auto launch = [&](auto stream_v) {
      constexpr bool SV = decltype(stream_v)::value;
      if (rope) {
        if constexpr (HD <= 128) {
          auto kernel = alone ? attn_decode_work_rope_alone_kernel<HD, SV> : attn_decode_work_rope_kernel<HD, SV>;
          hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, PYRE_DECODE_LAUNCH_ARGS, *rope);
        }
      } else {
        auto kernel = alone ? attn_decode_work_alone_kernel<HD, SV> : attn_decode_work_kernel<HD, SV>;
        hipLaunchKernelGGL(kernel, grid, dim3(256), 0, stream, PYRE_DECODE_LAUNCH_ARGS);
      }
    };
    if (page_size <= 32) launch(std::true_type{});
    else launch(std::false_type{});
  });
#undef PYRE_DECODE_LAUNCH_ARGS
  PYRE_REQUIRE(rc == 0, "attn_decode_work_bf16: no kernel for head_dim %d", hd);
  return check_launch("attn_decode_work_bf16");
}

}  // namespace

extern "C" int pyre_attn_decode_work_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                                          const int* work, int capacity, const int* positions,
                                          const int* seq_of_token, const int* block_table, int table_stride,
                                          float* part_acc, float* part_ml, int* counters, int alone, int nq,
                                          int nkv, int hd, int page_size, float scale, int window,
                                          hipStream_t stream) {
  return launch_decode_work(q, out, const_cast<void*>(k_cache), const_cast<void*>(v_cache), work, capacity, positions,
                            seq_of_token, block_table, table_stride, part_acc, part_ml, counters, alone, nq, nkv, hd,
                            page_size, scale, window, nullptr, stream);
}

extern "C" int pyre_attn_decode_work_rope_supports(int hd, int page_size, int nq, int nkv, long partial_stride) {
  // one group of query heads per key/value head: no other block reads the position that a block writes
  return pyre_attn_mfma_supports(hd, page_size, nq, nkv) && hd <= 128 && nq / nkv <= 16 && partial_stride % 4 == 0;
}

extern "C" int pyre_attn_decode_work_rope_bf16(const float* qkv, int n_partials, long partial_stride, const void* bias,
                                               int bias_dt, const float* cos_t, const float* sin_t, const int* slots,
                                               int n_rows, int write_kv, void* out, void* k_cache, void* v_cache,
                                               const int* work, int capacity, const int* positions,
                                               const int* seq_of_token, const int* block_table, int table_stride,
                                               float* part_acc, float* part_ml, int* counters, int alone, int nq,
                                               int nkv, int hd, int page_size, float scale, int window,
                                               hipStream_t stream) {
  PYRE_REQUIRE(pyre_attn_decode_work_rope_supports(hd, page_size, nq, nkv, partial_stride),
               "attn_decode_work_rope_bf16: head_dim %d, page_size %d, heads %d/%d or partial sums %ld apart are not "
               "supported", hd, page_size, nq, nkv, partial_stride);
  PYRE_REQUIRE(qkv && n_partials >= 1 && cos_t && sin_t && n_rows > 0, "attn_decode_work_rope_bf16: no product or tables");
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "attn_decode_work_rope_bf16: unknown bias dtype");
  PYRE_REQUIRE(!write_kv || slots, "attn_decode_work_rope_bf16: keys and values to write, but no slots");
  PYRE_REQUIRE(reinterpret_cast<uintptr_t>(qkv) % 16 == 0 && reinterpret_cast<uintptr_t>(cos_t) % 16 == 0 &&
                   reinterpret_cast<uintptr_t>(sin_t) % 16 == 0 && (!bias || reinterpret_cast<uintptr_t>(bias) % 16 == 0),
               "attn_decode_work_rope_bf16: the product, its bias and the tables must lie on 16 bytes");
  const RopeIn rope{qkv, n_partials, partial_stride, bias, bias_dt, cos_t, sin_t, slots, n_rows, write_kv};
  return launch_decode_work(nullptr, out, k_cache, v_cache, work, capacity, positions, seq_of_token, block_table,
                            table_stride, part_acc, part_ml, counters, alone, nq, nkv, hd, page_size, scale, window,
                            &rope, stream);
}

extern "C" int pyre_attn_prefill_bf16(const void* q, void* out, const void* k_cache,
                                      const void* v_cache, const int* tiles, int n_tiles,
                                      const int* positions, const int* seq_of_token,
                                      const int* block_table, int table_stride, int nq, int nkv,
                                      int hd, int page_size, float scale, int window, hipStream_t stream) {
  PYRE_REQUIRE(pyre_attn_mfma_supports(hd, page_size, nq, nkv),
               "attn_prefill_bf16: head_dim %d (multiples of 32 up to 256), page_size %d (multiples of 16), "
               "heads %d/%d are not supported", hd, page_size, nq, nkv);
  PYRE_REQUIRE(table_stride > 0, "attn_prefill_bf16: bad table");
  if (n_tiles <= 0) return 0;
  const int hgroups = (nq / nkv + 3) / 4;
  PYRE_REQUIRE(nkv * hgroups <= 65535, "attn_prefill_bf16: grid too large");
  const dim3 grid(n_tiles, nkv * hgroups);
  const int rc = dispatch_head(hd, [&](auto HDc) {
    constexpr int HD = decltype(HDc)::value;
    hipLaunchKernelGGL(attn_prefill_kernel<HD>, grid, dim3(256), 0, stream, static_cast<const bf16*>(q),
                       static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache), static_cast<bf16*>(out),
                       tiles, positions, seq_of_token, block_table, table_stride, nq, nkv, page_size, scale * kLog2e,
                       window);
  });
  PYRE_REQUIRE(rc == 0, "attn_prefill_bf16: no kernel for head_dim %d", hd);
  return check_launch("attn_prefill_bf16");
}

extern "C" int pyre_attn_prefill_waves(int nq, int nkv) { return nq / nkv > 4 ? 8 : 4; }

extern "C" int pyre_attn_prefill_work_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                                           const int* work, int n_items, float* partials, int* counters,
                                           int n_slots, const int* positions, const int* seq_of_token, const int* block_table,
                                           int table_stride, int nq, int nkv, int hd, int page_size, float scale,
                                           int window, hipStream_t stream) {
  PYRE_REQUIRE(pyre_attn_mfma_supports(hd, page_size, nq, nkv) && hd <= 128,
               "attn_prefill_work_bf16: head_dim %d (multiples of 32 up to 128), page_size %d (multiples of 16), "
               "heads %d/%d are not supported", hd, page_size, nq, nkv);
  PYRE_REQUIRE(table_stride > 0 && n_slots >= 0, "attn_prefill_work_bf16: bad table or slots");
  PYRE_REQUIRE(reinterpret_cast<uintptr_t>(work) % 16 == 0, "attn_prefill_work_bf16: the work list must lie on 16 bytes");
  if (n_items <= 0) return 0;
  const int n_rep = nq / nkv;
  const int nw = pyre_attn_prefill_waves(nq, nkv);
  const int hgroups = (n_rep + nw - 1) / nw;
  PYRE_REQUIRE(n_items <= 65535, "attn_prefill_work_bf16: a list of %d blocks is too long for one launch", n_items);
  // the blocks of one row of the list are neighbours in the order of dispatch: the list's order is the order of starts
  const dim3 grid(nkv * hgroups, n_items);
#define PYRE_PREFILL_ARGS                                                                                          \
  static_cast<const bf16*>(q), static_cast<const bf16*>(k_cache), static_cast<const bf16*>(v_cache),               \
      static_cast<bf16*>(out), reinterpret_cast<const int4*>(work), partials, counters, n_slots, positions,        \
      seq_of_token, block_table, table_stride, nq, nkv, page_size, scale * kLog2e, window
  const int rc = dispatch_head(hd, [&](auto HDc) {
    constexpr int HD = decltype(HDc)::value;
    if constexpr (HD <= 128) {
      if (nw == 8)
        hipLaunchKernelGGL((attn_prefill_tile32_kernel<HD, 8>), grid, dim3(512), 0, stream, PYRE_PREFILL_ARGS);
      else
        hipLaunchKernelGGL((attn_prefill_tile32_kernel<HD, 4>), grid, dim3(256), 0, stream, PYRE_PREFILL_ARGS);
    }
  });
#undef PYRE_PREFILL_ARGS
  PYRE_REQUIRE(rc == 0, "attn_prefill_work_bf16: no kernel for head_dim %d", hd);
  return check_launch("attn_prefill_work_bf16");
}
