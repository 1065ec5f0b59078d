// out[m, n] = sum_k X[m, k] W[n, k] for 65 to 256 rows of X in bfloat16: the matrix products of
// a decode step of many requests (pyre/model.py:315-319,338-342 at the batch sizes of
// pyre/scheduler.py), where every weight is still read once but the arithmetic is no longer
// free. For products with few output columns (q/k/v, the attention output, the feed-forward's
// way down) the BLAS library's kernels take 19 us or more whatever the size; this kernel keeps
// all rows of X of a step against 64 rows of W and splits k over blocks instead.
//
// The product is computed transposed, out^T = W X^T, on MFMA 32x32x16: A = 32 rows of W, B = 32
// rows of X, both read along k as they are stored. A block owns 64 rows of W and BM = 128 or
// 256 rows of X: four multiplying waves (wave w the rows 32 CW w .. of X, CW = 1 or 2 tiles,
// against both tiles of W) and a fifth that loads W. k is walked in stages of 32 through two
// rings in LDS, one of W and one of X, that are filled by loads from memory straight into LDS
// several stages ahead; a stage holds its rows as 64-byte rows whose four 16-byte pieces are
// exchanged among themselves by the row's number, so that the operand reads of 32 lanes (32
// rows, the same k) spread over all banks. One barrier per stage: it publishes the stage that
// has landed and frees the one before it.
//
// `ksplit` blocks share rows of W (grid.y); each writes a partial sum, float32 [ksplit][M][N],
// that the consumer adds in the order 0..ksplit-1. The order of an element's sums is a
// function of k alone: a row's result does not depend on the other rows of the step or on
// their number. The time is set by how many bytes a block has on their way at once (the rows of
// X come from L2 again for every 64 rows of W): it pays where ksplit can fill the chip in one
// round of blocks, which the caller checks.
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BN = 64;   // rows of W per block
constexpr int BK = 32;   // k per stage: rows of 64 bytes

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

// SW, SX: stages in the rings of W and of X. The weights come from memory (about 2 us away), the
// rows of X from L2 (well under 1 us): W is loaded by a fifth wave of its own, whose loads
// can then run far ahead without holding up the others' (a wave's loads finish in order).
template <int CW, int SW, int SX>
__global__ __launch_bounds__(320, 2) void gemm_mid_kernel(const bf16* __restrict__ X, size_t ldx,
                                                          const bf16* __restrict__ W, size_t ldw,
                                                          float* __restrict__ out, int M, int N, int K, int kper) {
  constexpr int BM = 128 * CW, WSTAGE = BN * 64, XSTAGE = BM * 64;
  constexpr int PERW = BN / 16;      // loads of 16 rows per stage of W, all by the loading wave
  constexpr int PERX = BM / 16 / 4;  // and of X, per multiplying wave
  __shared__ __attribute__((aligned(1024))) unsigned char lds[SW * WSTAGE + SX * XSTAGE];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int c = lane & 31, half = lane >> 5;
  const int ks = blockIdx.y, kbeg = ks * kper, kend = min(K, kbeg + kper);
  const int stages = (kend - kbeg + BK - 1) / BK;
  const unsigned lds_base = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds)));
  const bf16* zero = reinterpret_cast<const bf16*>(kZeroPiece);
  // A load of 16 rows: the piece that lands at row lane / 4 of them, place lane % 4, is piece
  // (place ^ swizzle of the row) of the row's 32 k. Rows past the end are zeros.
  const int place_row = lane >> 2;

  if (wave == 4) {
    // ---- the loading wave: 64 rows of W per stage.
    const bf16* src[PERW];
    int kofs[PERW];
#pragma unroll
    for (int i = 0; i < PERW; ++i) {
      const int row = 16 * i + place_row;
      kofs[i] = 8 * ((lane & 3) ^ ((row >> 2) & 3));
      const int n = blockIdx.x * BN + row;
      src[i] = n < N ? W + static_cast<size_t>(n) * ldw + kbeg + kofs[i] : nullptr;
    }
    auto issue = [&](int st, int slot) {
      const int left = st < stages ? kend - kbeg - BK * st : 0;  // k of this part from the stage's start on
#pragma unroll
      for (int i = 0; i < PERW; ++i)
        load_to_lds(src[i] && kofs[i] < left ? src[i] + BK * st : zero, lds_base + slot * WSTAGE + i * 1024);
    };
#pragma unroll
    for (int st = 0; st < SW - 1; ++st) issue(st, st);
    int slot = 0;
    for (int st = 0; st < stages; ++st) {
      wait_loads<PERW * (SW - 2)>();  // loads finish in the order of issue: stage st is there
      __syncthreads();                // the others know, and have multiplied stage st - 1
      issue(st + SW - 1, slot == 0 ? SW - 1 : slot - 1);
      slot = slot + 1 == SW ? 0 : slot + 1;
    }
    wait_loads<0>();  // the loads past the end
    return;
  }

  // ---- the multiplying waves: wave w loads a quarter of the rows of X and multiplies its own
  // 32 CW rows of them against the block's 64 rows of W.
  const bf16* src[PERX];
  int kofs[PERX];
#pragma unroll
  for (int i = 0; i < PERX; ++i) {
    const int row = 16 * (wave + 4 * i) + place_row;
    kofs[i] = 8 * ((lane & 3) ^ ((row >> 2) & 3));
    src[i] = row < M ? X + static_cast<size_t>(row) * ldx + kbeg + kofs[i] : nullptr;
  }
  const unsigned x_base = lds_base + SW * WSTAGE;
  auto issue = [&](int st, int slot) {
    const int left = st < stages ? kend - kbeg - BK * st : 0;
#pragma unroll
    for (int i = 0; i < PERX; ++i)
      load_to_lds(src[i] && kofs[i] < left ? src[i] + BK * st : zero, x_base + slot * XSTAGE + (wave + 4 * i) * 1024);
  };

  f32x16 acc[2][CW];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < CW; ++ct)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[rt][ct][i] = 0.f;

  const int swz = (c >> 2) & 3;
  const int xrow0 = 32 * CW * wave + c;  // this lane's row of X, for tile 0
#pragma unroll
  for (int st = 0; st < SX - 1; ++st) issue(st, st);
  int wslot = 0, xslot = 0;
  for (int st = 0; st < stages; ++st) {
    wait_loads<PERX * (SX - 2)>();  // this wave's share of stage st of X is there
    __syncthreads();                // and everyone's, and stage st of W; and everyone has multiplied stage st - 1
    issue(st + SX - 1, xslot == 0 ? SX - 1 : xslot - 1);
    const unsigned char* wb = lds + wslot * WSTAGE;
    const unsigned char* xb = lds + SW * WSTAGE + xslot * XSTAGE;
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const int piece = 16 * ((2 * kk + half) ^ swz);
      bf16x8 a[2], b[CW];
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) a[rt] = *reinterpret_cast<const bf16x8*>(wb + (32 * rt + c) * 64 + piece);
#pragma unroll
      for (int ct = 0; ct < CW; ++ct) b[ct] = *reinterpret_cast<const bf16x8*>(xb + (xrow0 + 32 * ct) * 64 + piece);
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < CW; ++ct)
          acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[rt], b[ct], acc[rt][ct], 0, 0, 0);
    }
    wslot = wslot + 1 == SW ? 0 : wslot + 1;
    xslot = xslot + 1 == SX ? 0 : xslot + 1;
  }
  wait_loads<0>();  // the loads past the end

  // acc[rt][ct][4 q + j]: row 32 rt + 8 q + 4 half + j of the block's tile of W, row
  // 32 (CW wave + ct) + c of X.
  float* o = out + static_cast<size_t>(ks) * M * N;
  const bool vec = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
  for (int ct = 0; ct < CW; ++ct) {
    const int m = 32 * (CW * wave + ct) + c;
    if (m >= M) continue;
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int n = blockIdx.x * BN + 32 * rt + 8 * q + 4 * half;
        if (n >= N) continue;
        float* dst = o + static_cast<size_t>(m) * N + n;
        if (vec && n + 3 < N) {
          *reinterpret_cast<f32x4*>(dst) =
              f32x4{acc[rt][ct][4 * q], acc[rt][ct][4 * q + 1], acc[rt][ct][4 * q + 2], acc[rt][ct][4 * q + 3]};
        } else {
          for (int j = 0; j < 4 && n + j < N; ++j) dst[j] = acc[rt][ct][4 * q + j];
        }
      }
  }
}

int check_mid(const char* name, const void* X, const void* W, int M, int N, int K, long ldx, long ldw) {
  PYRE_REQUIRE(pyre_gemm_mid_supports(M, N, K, ldx, ldw),
               "%s: M=%d (1..256) N=%d K=%d (multiples of 8) ldx=%ld ldw=%ld (multiples of 8, >= K) are not supported",
               name, M, N, K, ldx, ldw);
  PYRE_REQUIRE(reinterpret_cast<uintptr_t>(X) % 16 == 0 && reinterpret_cast<uintptr_t>(W) % 16 == 0,
               "%s: operands must lie on 16 bytes", name);
  return 0;
}

}  // namespace

extern "C" int pyre_gemm_mid_supports(int M, int N, int K, long ldx, long ldw) {
  return M >= 1 && M <= 256 && N >= 1 && K >= 8 && K % 8 == 0 && ldx >= K && ldx % 8 == 0 && ldw >= K && ldw % 8 == 0;
}

// out: float32 [ksplit][M][N].
extern "C" int pyre_gemm_mid_bf16(const void* X, long ldx, const void* W, long ldw, float* out, int M, int N,
                                  int K, int ksplit, hipStream_t stream) {
  if (int rc = check_mid("gemm_mid_bf16", X, W, M, N, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(ksplit >= 1 && ksplit <= 64, "gemm_mid_bf16: ksplit=%d", ksplit);
  const int kper = ((K + ksplit - 1) / ksplit + BK - 1) / BK * BK;
  PYRE_REQUIRE(static_cast<long>(ksplit - 1) * kper < K, "gemm_mid_bf16: a part of k would be empty (K=%d, ksplit=%d)", K, ksplit);
  const dim3 grid((N + BN - 1) / BN, ksplit);
  const bf16* x = static_cast<const bf16*>(X);
  const bf16* w = static_cast<const bf16*>(W);
  if (M > 128) {
    hipLaunchKernelGGL((gemm_mid_kernel<2, 7, 3>), grid, dim3(320), 0, stream, x, static_cast<size_t>(ldx), w,
                       static_cast<size_t>(ldw), out, M, N, K, kper);
  } else {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 8, 4>), grid, dim3(320), 0, stream, x, static_cast<size_t>(ldx), w,
                       static_cast<size_t>(ldw), out, M, N, K, kper);
  }
  return check_launch("gemm_mid_bf16");
}
