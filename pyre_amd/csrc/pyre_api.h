// C entry points of the gfx950 kernel library. Pointers are device pointers
// unless a comment says otherwise; `stream` is the HIP stream the work is put on.
// Every function returns 0, or non-zero after storing a message that
// pyre_last_error() returns. Element type codes: 0 = float32, 1 = bfloat16.
#pragma once

#include <hip/hip_runtime.h>

extern "C" {

const char* pyre_last_error();
int pyre_abi_version();
// Compute units of the current device (256 where there is no device to ask): the kernels whose
// blocks are meant to fill the chip in one round shape their launches by it, and so must
// whoever plans work for them on the host.
int pyre_compute_units();
// A digest of the sources this library was compiled from, as the build wrote it in.
const char* pyre_sources_digest();

// Streams `bytes` of device memory through the chip and writes (almost) nothing:
// a measurement of achievable read bandwidth.
int pyre_read_probe(const void* p, size_t bytes, int blocks, unsigned* sink, hipStream_t stream);

int pyre_embed(const void* table, int table_dt, const int* ids, float* out, int n, int hidden,
               hipStream_t stream);

int pyre_add_rmsnorm(float* resid, const void* delta, int delta_dt, int n_partials,
                     long partial_stride, const void* bias, int bias_dt, const void* gain,
                     int gain_dt, void* out, int out_dt, const int* rows, int n, int hidden,
                     float eps, hipStream_t stream);

// Finishes the q/k/v product (partial sums, bias), rotates queries and keys by position, stores
// the queries and, with write_kv, keys and values at slots[n] = page * page_size + offset
// (-1: not stored) of caches k [pages, nkv, page_size, hd] and v [pages, nkv, hd, page_size]. The
// tokens that one call writes into one page are neighbours in the batch and take consecutive
// slots in rising order (a request's next positions); the last of them zeroes the values of the
// slots behind it, so that nothing of the page's previous owner stays behind a request's last key.
int pyre_rope_kv_write(const void* qkv, int qkv_dt, int n_partials, long partial_stride,
                       const void* bias, int bias_dt, void* q_out, int q_dt, void* k_cache,
                       void* v_cache, int cache_dt, const float* cos_t, const float* sin_t,
                       int rotary_dim, const int* positions, const int* slots, int n, int nq,
                       int nkv, int hd, int page_size, int write_kv, hipStream_t stream);

int pyre_silu_mul(const void* gu, int gu_dt, int n_partials, long partial_stride, void* out,
                  int out_dt, int n, int inter, hipStream_t stream);

int pyre_reduce_partials(const void* in, int in_dt, int n_partials, long partial_stride,
                         const void* bias, int bias_dt, void* out, int out_dt, int n, int width,
                         hipStream_t stream);

int pyre_gemm_generic(const void* A, int a_dt, long lda, const int* a_rows, const void* W,
                      int w_dt, long ldw, const void* bias, int bias_dt, void* out, int out_dt,
                      long ldo, int M, int N, int K, hipStream_t stream);

// base[o][ids[i]][0 .. row_elems) = pattern for every o < n_outer: rows of a contiguous
// [n_outer, n_rows, row_elems] tensor of 2- or 4-byte elements (outer_stride in elements).
// ids_host is HOST memory. Zeroes state slots; poisons freed pages in the debug mode.
int pyre_fill_rows(void* base, int elem_bytes, long outer_stride, int n_outer, int n_rows, long row_elems,
                   const int* ids_host, int n_ids, unsigned pattern, hipStream_t stream);

// The same for float32 operands and results only, on the matrix cores' float32 instruction:
// the product of the true 32-bit path. The order of an element's additions depends on k alone.
// ksplit > 1: partial sums out[s] (part_stride elements apart) over ksplit parts of k, the bias
// in part 0; the consumer adds them in the order 0..ksplit-1.
int pyre_gemm_f32(const float* A, long lda, const float* W, long ldw, const void* bias, int bias_dt,
                  float* out, long ldo, long part_stride, int M, int N, int K, int ksplit,
                  hipStream_t stream);

// bfloat16 products with 1..64 rows (decode): 1 if the kernel takes the shape.
int pyre_gemm_skinny_supports(int M, int N, int K, long ldx, long ldw);

// out: float32 [ksplit][M][N] partial sums of X[M, K] W[N, K]^T over ksplit parts of k.
int pyre_gemm_skinny_bf16(const void* X, long ldx, const void* W, long ldw, float* out, int M, int N,
                          int K, int ksplit, hipStream_t stream);

// W = [gate rows; up rows] (two_i x K); out: bfloat16 [M][two_i / 2] = silu(X gate^T) * (X up^T).
int pyre_gemm_skinny_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M,
                               int two_i, int K, hipStream_t stream);

// The first of them for up to 256 rows (a decode step of many requests), for products with few
// output columns: a block keeps all rows of X against 64 rows of W (128 with `wide`), and ksplit
// blocks share them. out: float32 [ksplit][M][N].
int pyre_gemm_mid_supports(int M, int N, int K, long ldx, long ldw);
int pyre_gemm_mid_bf16(const void* X, long ldx, const void* W, long ldw, float* out, int M, int N, int K,
                       int ksplit, int wide, hipStream_t stream);
// The second of them for up to 256 rows: a block takes 64 or 96 features (pyre_gemm_mid_silu_blocks
// blocks in all) against all rows of X; it pays where one round of blocks holds them.
int pyre_gemm_mid_silu_blocks(int M, int two_i);
int pyre_gemm_mid_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M, int two_i,
                            int K, hipStream_t stream);

// tokens: the n tokens of the flat batch to attend for, or null for tokens 0..n-1. max_keys: a
// bound on the keys that any of them sees (the block table's width in tokens will do); part:
// n * nq * pyre_attn_generic_spans(max_keys) * (hd + 2) floats of scratch when that is more than one span.
// matrix_cores: float32 queries and caches with a head size of 16, 32, ..., 128 and pages of a multiple
// of 16 tokens go to the kernel that reads a span's keys and values once for all query heads of a
// key/value head and multiplies on the float32 matrix instruction (its sums run in another order than
// those of one block per head, which 0 asks for: a difference of rounding). Which kernel runs depends
// on these sizes alone, never on the tokens of the call.
int pyre_attn_generic_spans(int max_keys);
int pyre_attn_generic(const void* q, void* out, int q_dt, const void* k_cache,
                      const void* v_cache, int cache_dt, const int* tokens, const int* positions,
                      const int* seq_of_token, const int* block_table, int table_stride, int n,
                      int nq, int nkv, int hd, int page_size, float scale, int window, int max_keys,
                      float* part, int matrix_cores, hipStream_t stream);

// Prompt portions in true float32 on the matrix cores' float32 instruction: tiles as for
// pyre_attn_prefill_bf16, float32 queries, caches and output, any head size up to 256, any
// page size. The order of a token's sums depends on its own bounds alone.
int pyre_attn_prefill_f32(const float* q, float* out, const float* k_cache, const float* v_cache,
                          const int* tiles, int n_tiles, const int* positions, const int* seq_of_token,
                          const int* block_table, int table_stride, int nq, int nkv, int hd, int page_size,
                          float scale, int window, hipStream_t stream);

// 1 if the MFMA attention kernels take this geometry (else use pyre_attn_generic).
int pyre_attn_mfma_supports(int hd, int page_size, int nq, int nkv);

// One new token per request, from a work list that deals every request's keys to blocks of
// four waves:
// rows of eight ints: work[0] = (blocks in the list, 0, ...), work[1 + i] = (token in the flat batch,
// block b of its request + 65536 * blocks nb of its request (<= 64), chunks `per` of 32 keys that a
// wave of this request takes, the request's first partial slot, the token's position, its request's
// row of the block table, 0, 0: the kernel takes position and row from the list, `positions` and
// `seq_of_token` are not read); block b takes chunks 4 b per ..
// 4 (b + 1) per - 1 of its request, counted from the first chunk that the token sees, and the
// nb blocks of a request cover all of them. The slots of the requests are disjoint runs of nb
// within 0..capacity-1. `alone`: a compute unit runs one block at a time (for steps of so few
// requests that a block per unit covers them); else two. The launch has
// `capacity` blocks per key/value head (and group of 16 query heads); blocks past the list's
// end exit. Scratch: part_acc [capacity, items, 16, hd] and part_ml [capacity, items, 16, 2]
// floats, counters [capacity, items] ints that are zero before the first call and are left
// at zero, items = nkv * ceil(nq / nkv / 16).
int pyre_attn_decode_work_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                               const int* work, int capacity, const int* positions,
                               const int* seq_of_token, const int* block_table, int table_stride,
                               float* part_acc, float* part_ml, int* counters, int alone, int nq, int nkv,
                               int hd, int page_size, float scale, int window, hipStream_t stream);

// The same for a step of single tokens straight from the step's q/k/v product (float32 partial sums
// [n_partials][n_rows][(nq + 2 nkv) hd], partial_stride elements apart, with its bias or null): every
// block sums, biases and rotates its heads' queries itself, and for every token and key/value head one
// wave writes the token's rotated key and its value into the cache (slots[token], -1: not stored;
// write_kv 0: a layer that keeps none) and zeroes the values behind it in its page, all with the
// arithmetic of pyre_rope_kv_write (the same bits in the cache and in the result), so that no kernel
// runs between the product and the attention. Full-head rotation (cos_t, sin_t: [positions][hd / 2]),
// heads of up to 128 elements, up to 16 query heads per key/value head.
int pyre_attn_decode_work_rope_supports(int hd, int page_size, int nq, int nkv, long partial_stride);
int pyre_attn_decode_work_rope_bf16(const float* qkv, int n_partials, long partial_stride, const void* bias,
                                    int bias_dt, const float* cos_t, const float* sin_t, const int* slots,
                                    int n_rows, int write_kv, void* out, void* k_cache, void* v_cache,
                                    const int* work, int capacity, const int* positions, const int* seq_of_token,
                                    const int* block_table, int table_stride, float* part_acc, float* part_ml,
                                    int* counters, int alone, int nq, int nkv, int hd, int page_size, float scale,
                                    int window, hipStream_t stream);


// Prompt portions. tiles[i] = (first token in the flat batch, token count <= 32),
// all tokens of a tile from one request at consecutive positions. Every wave reads the
// cache directly (any head size that pyre_attn_mfma_supports takes).
int pyre_attn_prefill_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                           const int* tiles, int n_tiles, const int* positions,
                           const int* seq_of_token, const int* block_table, int table_stride,
                           int nq, int nkv, int hd, int page_size, float scale, int window,
                           hipStream_t stream);

// The same for heads of up to 128 elements from a work list: K and V go straight into LDS in
// chunks of 64 keys for 32x32 MFMA tiles, and the chunks of a tile may be dealt to several blocks.
// work[2 i] = (first token of the tile, tokens <= 32, first chunk, last chunk), work[2 i + 1] =
// (first partial slot of the tile, this block's number among the tile's blocks, their number
// nb, 0); the nb blocks of a tile cover the chunks lo / 64 .. hi / 64 of the keys lo .. hi that
// its tokens see, each chunk once. A block has pyre_attn_prefill_waves(nq, nkv) waves, one per
// query head of a key/value head (groups of that many heads: `groups`). Scratch for tiles
// of more than one block: partials [slots, nkv * groups, waves, hd / 32 * 1024 + 128] floats
// and counters [slots, nkv * groups, waves] ints that are zero before the first call and are
// left at zero.
int pyre_attn_prefill_waves(int nq, int nkv);
int pyre_attn_prefill_work_bf16(const void* q, void* out, const void* k_cache, const void* v_cache,
                                const int* work, int n_items, float* partials, int* counters,
                                int n_slots, const int* positions, const int* seq_of_token, const int* block_table,
                                int table_stride, int nq, int nkv, int hd, int page_size, float scale,
                                int window, hipStream_t stream);

// scratch: m * 64 floats followed by m * 64 ints of device memory.
int pyre_argmax(const float* logits, long row_stride, int* out, void* scratch, int m, int vocab,
                hipStream_t stream);

// pyre_argmax without a scratch argument and without any allocation. It has no counterpart in
// the reference; it is for callers that cannot allocate device memory: code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc. The slices' partial results
// go to an array that is part of the library's device image (128 KB on every GPU the library
// runs on, until the process ends), so m is at most PYRE_ARGMAX_STATIC_MAX_ROWS; more rows are
// refused with an error. The caller makes the GPU of `stream`, `logits` and `out` the current
// device. Same kernels and same results as pyre_argmax. All calls on one GPU share that GPU's
// array: calls that may overlap there (two streams, two threads) race; put them on one stream
// or use pyre_argmax with scratch of their own. The first call on a device looks the array's
// address up (hipGetSymbolAddress), which must not happen while a stream is capturing: a caller
// that captures calls pyre_argmax_static_init() on that device beforehand (it launches nothing
// and may be called any number of times).
#define PYRE_ARGMAX_STATIC_MAX_ROWS 256
int pyre_argmax_static_init();
int pyre_argmax_static(const float* logits, long row_stride, int* out, int m, int vocab,
                       hipStream_t stream);

// tokens[i] = ids[src[i]] where src[i] >= 0: a step's token that is the previous step's
// sampled id, taken on the device so that the host need not wait for it.
int pyre_feed_tokens(int* tokens, const int* src, const int* ids, int n, hipStream_t stream);

int pyre_sample(const float* logits, long row_stride, const float* temperature,
                const float* uniform, int* out, int m, int vocab, hipStream_t stream);

}  // extern "C"
