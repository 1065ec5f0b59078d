// out[m, n] = sum_k X[m, k] W[n, k] for up to 256 rows of X in bfloat16: the matrix products of
// a decode step (pyre/model.py:315-319,338-342 at the batch sizes of pyre/scheduler.py), above all
// of many requests, where every weight is still read once but the arithmetic is no longer
// free. For products with few output columns (q/k/v, the attention output, the feed-forward's
// way down) the BLAS library's kernels take 19 us or more whatever the size; this kernel keeps
// all rows of X of a step against 64 rows of W and splits k over blocks instead.
//
// The product is computed transposed, out^T = W X^T, on MFMA 32x32x16: A = 32 rows of W, B = 32
// rows of X, both read along k as they are stored. A block owns 64 RW rows of W and BM = 32 to 256
// rows of X: RW groups of XW = 1 to 4 multiplying waves (a group on 64 rows of W, its wave q
// on the rows 32 CW q .. of X, CW = 1 or 2 tiles, against both tiles of W) and some waves that only
// load. k is walked in stages of 64 through a ring in LDS that is filled by loads from memory
// straight into LDS, S - 1 stages ahead; a stage holds its rows as 128-byte rows whose eight
// 16-byte pieces are exchanged among themselves by the row's number, so that the operand reads
// of 32 lanes (32 rows, the same k) spread over all banks. One barrier per stage: it publishes
// the stage that has landed and frees the one before it.
//
// kPartials: `ksplit` blocks share rows of W (grid.y); each writes a partial sum, float32
// [ksplit][M][N], that the consumer adds in the order 0..ksplit-1. kSiluMul (W = gate rows, then
// up rows; ksplit = 1): bfloat16 silu(gate) * up, [M][N / 2]. The order of an element's sums
// is a function of k alone: a row's result does not depend on the other rows of the step or on
// their number. The time is set by the bytes a compute unit can take from L2 (the rows of X
// come again for every block): it pays where the blocks fill the chip in one round, which the
// caller checks.
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BN = 64;   // rows of W per block
constexpr int BK = 64;   // k per stage: rows of 128 bytes

// 16 bytes per lane from global memory straight into LDS: lane x's piece lands at
// lds_addr + 16 x. The compiler does not know of these loads; whoever reads the bytes
// waits for them with wait_loads (they finish in the order of issue) and a barrier.
__device__ inline void load_to_lds(const void* src, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory", "m0");
}
// The same for bytes that are read once (the weights): past the caches.
__device__ inline void load_to_lds_once(const void* src, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off nt" : : "v"(src), "s"(lds_addr) : "memory", "m0");
}
template <int N>
__device__ inline void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __attribute__((aligned(16))) const unsigned kZeroPiece[4] = {0u, 0u, 0u, 0u};

enum Epilogue { kPartials = 0, kSiluMul = 1 };

// RW groups of XW multiplying waves, each group on 64 rows of W, and NL waves that only load; S
// stages in the ring. What a wave can have loaded per microsecond is limited (about 9 GB/s from
// L2, whatever the pattern and however many loads it has on their way; a compute unit takes
// about 84 GB/s), so the loads of a stage are dealt to all waves, and there are more waves than
// multiply; a stage is the 64 RW rows of W, then the BM rows of X. kSiluMul: a group's 64 rows
// are 32 gate rows and the up rows of the same features, so that a lane holds both for its
// elements; out is bfloat16 [M][N / 2].
template <int CW, int XW, int RW, int EPI, int NL, int S>
__global__ __launch_bounds__(64 * (XW * RW + NL)) void gemm_mid_kernel(const bf16* __restrict__ X, size_t ldx,
                                                                      const bf16* __restrict__ W, size_t ldw,
                                                                      void* __restrict__ out, int M, int N, int K,
                                                                      int kper) {
  constexpr int BM = 32 * CW * XW, BW = BN * RW, ROWS = BW + BM, STAGE = ROWS * 128;
  constexpr int NWAVES = XW * RW + NL, LOADS = ROWS / 8;
  constexpr int PER = (LOADS + NWAVES - 1) / NWAVES;  // loads of 8 rows per wave and stage
  // Where the loads of a stage do not divide evenly over the waves, the spare turns load zeros
  // into a kilobyte behind the ring, so that every wave counts the same number of loads.
  constexpr bool SPARE = LOADS % NWAVES != 0;
  __shared__ __attribute__((aligned(1024))) unsigned char lds[S * STAGE + (SPARE ? 1024 : 0)];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
  const int c = lane & 31, half = lane >> 5;
  const int ks = blockIdx.y, kbeg = ks * kper, kend = min(K, kbeg + kper);
  const int stages = (kend - kbeg + BK - 1) / BK;
  const int inter = N / 2;

  // Every wave loads: of load j = wave + NWAVES i (rows 8 j .. 8 j + 7 of the stage) this lane
  // brings the piece that lands at row 8 j + lane / 8, place lane % 8, which is piece
  // (place ^ swizzle of the row) of the row's 64 k. Rows past the end are zeros.
  const unsigned lds_base = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(lds)));
  const bf16* zero = reinterpret_cast<const bf16*>(kZeroPiece);
  const bf16* src[PER];
  int kofs[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int row = 8 * (wave + NWAVES * i) + (lane >> 3);
    kofs[i] = 8 * ((lane & 7) ^ ((row >> 1) & 7));
    const bf16* base = nullptr;
    if (row >= ROWS) {
      // a spare turn
    } else if (row < BW) {
      int n;  // the row of W behind row `row` of the block's tile, or past the end
      if (EPI == kSiluMul) {
        const int f = blockIdx.x * (32 * RW) + 32 * (row >> 6) + (row & 31);
        n = f < inter ? ((row >> 5) & 1) * inter + f : N;
      } else {
        n = blockIdx.x * BW + row;
      }
      if (n < N) base = W + static_cast<size_t>(n) * ldw;
    } else if (row - BW < M) {
      base = X + static_cast<size_t>(row - BW) * ldx;
    }
    src[i] = base ? base + kbeg + kofs[i] : nullptr;
  }
  auto issue = [&](int st, int slot) {
    const int left = st < stages ? kend - kbeg - BK * st : 0;  // k of this part from the stage's start on
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int j = wave + NWAVES * i;  // rows 8 j .. of the stage: of W up to BW / 8
      const bf16* from = src[i] && kofs[i] < left ? src[i] + BK * st : zero;
      const unsigned to = j < LOADS ? lds_base + slot * STAGE + j * 1024 : lds_base + S * STAGE;
      if (j < BW / 8) load_to_lds_once(from, to);
      else load_to_lds(from, to);
    }
  };
#pragma unroll
  for (int st = 0; st < S - 1; ++st) issue(st, st);

  if (wave >= XW * RW) {
    // ---- a wave that only loads
    int slot = 0;
    for (int st = 0; st < stages; ++st) {
      wait_loads<PER * (S - 2)>();  // loads finish in the order of issue: this wave's share of stage st is there
      __syncthreads();              // everyone knows, and stage st - 1 has been multiplied
      issue(st + S - 1, slot == 0 ? S - 1 : slot - 1);
      slot = slot + 1 == S ? 0 : slot + 1;
    }
    wait_loads<0>();  // the loads past the end
    return;
  }

  // ---- a multiplying wave: its own 32 CW rows of X against its group's 64 rows of W.
  const int group = wave / XW, quarter = wave % XW;
  f32x16 acc[2][CW];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt)
#pragma unroll
    for (int ct = 0; ct < CW; ++ct)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[rt][ct][i] = 0.f;

  const int swz = (c >> 1) & 7;
  const int wrow0 = 64 * group + c;                // this lane's row of W in the stage, for tile 0
  const int xrow0 = BW + 32 * CW * quarter + c;    // and of X
  int slot = 0;
  for (int st = 0; st < stages; ++st) {
    wait_loads<PER * (S - 2)>();  // this wave's share of stage st is there
    __syncthreads();              // and everyone's; and everyone has multiplied stage st - 1
    issue(st + S - 1, slot == 0 ? S - 1 : slot - 1);
    const unsigned char* sb = lds + slot * STAGE;
    // The operands of step kk + 1 are read from LDS while step kk is multiplied.
    bf16x8 a[2], b[CW], an[2], bn[CW];
    auto read = [&](int kk, bf16x8 (&ra)[2], bf16x8 (&rb)[CW]) {
      const int piece = 16 * ((2 * kk + half) ^ swz);
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) ra[rt] = *reinterpret_cast<const bf16x8*>(sb + (wrow0 + 32 * rt) * 128 + piece);
#pragma unroll
      for (int ct = 0; ct < CW; ++ct) rb[ct] = *reinterpret_cast<const bf16x8*>(sb + (xrow0 + 32 * ct) * 128 + piece);
    };
    read(0, a, b);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      if (kk + 1 < BK / 16) read(kk + 1, an, bn);
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int ct = 0; ct < CW; ++ct)
          acc[rt][ct] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[rt], b[ct], acc[rt][ct], 0, 0, 0);
#pragma unroll
      for (int rt = 0; rt < 2; ++rt) a[rt] = an[rt];
#pragma unroll
      for (int ct = 0; ct < CW; ++ct) b[ct] = bn[ct];
    }
    slot = slot + 1 == S ? 0 : slot + 1;
  }
  wait_loads<0>();  // the loads past the end

  // acc[rt][ct][4 q + j]: row 32 rt + 8 q + 4 half + j of the group's tile of W, row
  // 32 (CW quarter + ct) + c of X.
  if (EPI == kPartials) {
    float* o = static_cast<float*>(out) + static_cast<size_t>(ks) * M * N;
    const bool vec = (N & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
#pragma unroll
    for (int ct = 0; ct < CW; ++ct) {
      const int m = 32 * (CW * quarter + ct) + c;
      if (m >= M) continue;
#pragma unroll
      for (int rt = 0; rt < 2; ++rt)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int n = blockIdx.x * BW + 64 * group + 32 * rt + 8 * q + 4 * half;
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
  } else {
    bf16* o = static_cast<bf16*>(out);
    const bool vec = (inter & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0;
#pragma unroll
    for (int ct = 0; ct < CW; ++ct) {
      const int m = 32 * (CW * quarter + ct) + c;
      if (m >= M) continue;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int f = blockIdx.x * (32 * RW) + 32 * group + 8 * q + 4 * half;
        if (f >= inter) continue;
        float y[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float gate = acc[0][ct][4 * q + j], up = acc[1][ct][4 * q + j];
          y[j] = gate / (1.f + __expf(-gate)) * up;
        }
        bf16* dst = o + static_cast<size_t>(m) * inter + f;
        if (vec && f + 3 < inter) {
          *reinterpret_cast<uint2*>(dst) = uint2{pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3])};
        } else {
          for (int j = 0; j < 4 && f + j < inter; ++j) dst[j] = from_float<bf16>(y[j]);
        }
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
                                  int K, int ksplit, int wide, hipStream_t stream) {
  if (int rc = check_mid("gemm_mid_bf16", X, W, M, N, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(ksplit >= 1 && ksplit <= 64, "gemm_mid_bf16: ksplit=%d", ksplit);
  const int kper = ((K + ksplit - 1) / ksplit + BK - 1) / BK * BK;
  PYRE_REQUIRE(static_cast<long>(ksplit - 1) * kper < K, "gemm_mid_bf16: a part of k would be empty (K=%d, ksplit=%d)", K, ksplit);
  const dim3 grid((N + BN - 1) / BN, ksplit);
  const bf16* x = static_cast<const bf16*>(X);
  const bf16* w = static_cast<const bf16*>(W);
  if (wide) {
    // Twice the rows of W a block, over half as much of k where the caller splits k further: a
    // block's bytes (its rows of W and all rows of X, over its part of k) are fewest where the two
    // are equally many, and at few rows of X a stage (and the barrier that goes with it) carries
    // twice the bytes. Measured on the 7B shape's way down, weights from memory: 25.6 us at 64
    // rows of X where 64 rows of W a block take 29.8 and the weight-streaming kernel 31.9.
    const dim3 grid2((N + 2 * BN - 1) / (2 * BN), ksplit);
    if (M <= 32) {
      hipLaunchKernelGGL((gemm_mid_kernel<1, 1, 2, kPartials, 8, 6>), grid2, dim3(64 * 10), 0, stream, x,
                         static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
    } else if (M <= 64) {
      hipLaunchKernelGGL((gemm_mid_kernel<1, 2, 2, kPartials, 8, 5>), grid2, dim3(64 * 12), 0, stream, x,
                         static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
    } else if (M <= 128) {
      hipLaunchKernelGGL((gemm_mid_kernel<1, 4, 2, kPartials, 8, 4>), grid2, dim3(64 * 16), 0, stream, x,
                         static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
    } else if (M <= 192) {
      hipLaunchKernelGGL((gemm_mid_kernel<2, 3, 2, kPartials, 8, 3>), grid2, dim3(64 * 14), 0, stream, x,
                         static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
    } else {
      hipLaunchKernelGGL((gemm_mid_kernel<2, 4, 2, kPartials, 8, 3>), grid2, dim3(64 * 16), 0, stream, x,
                         static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
    }
  } else if (M > 192) {
    hipLaunchKernelGGL((gemm_mid_kernel<2, 4, 1, kPartials, 6, 3>), grid, dim3(64 * 10), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
  } else if (M > 128) {
    hipLaunchKernelGGL((gemm_mid_kernel<2, 3, 1, kPartials, 6, 4>), grid, dim3(64 * 9), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
  } else if (M <= 32) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 1, 1, kPartials, 8, 6>), grid, dim3(64 * 9), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
  } else if (M <= 64) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 2, 1, kPartials, 8, 5>), grid, dim3(64 * 10), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
  } else {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 4, 1, kPartials, 8, 4>), grid, dim3(64 * 12), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, N, K, kper);
  }
  return check_launch("gemm_mid_bf16");
}

// W = [gate rows; up rows] (two_i x K); out: bfloat16 [M][two_i / 2] = silu(X gate^T) * (X up^T).
// A block takes 64 features (64 gate rows and 64 up rows, eight multiplying waves), or 96 with
// twelve for up to 128 rows of X (128 for 25 to 64 rows) where one round of blocks would not hold
// them otherwise. The
// rows of X that a block multiplies are 64, 96 (with 96 features), 128, 192 or 256, whichever
// holds M: fewer rows are fewer multiplying waves, fewer loads and a deeper ring (measured on the
// 7B shape, weights from memory: 49 us at 64 rows, 57 at 96, 63 at 128).
namespace {
int silu_features(int M, int two_i) {
  const int inter = two_i / 2, units = compute_units();
  if ((inter + 63) / 64 <= units || M > 128) return 64;
  // 128 features: the 32B shape's 27,648 in 216 blocks, for 25 to 64 rows of X (measured in its
  // decode steps against the weight-streaming kernel: 34.2 against 35.0 ms at 64 requests, 22.7
  // against 22.9 at 32, the same at 8, 13.0 against 12.7 at one)
  return M >= 25 && M <= 64 && (inter + 95) / 96 > units ? 128 : 96;
}
}  // namespace

extern "C" int pyre_gemm_mid_silu_blocks(int M, int two_i) {
  const int f = silu_features(M, two_i);
  return (two_i / 2 + f - 1) / f;
}

extern "C" int pyre_gemm_mid_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out, int M,
                                       int two_i, int K, hipStream_t stream) {
  if (int rc = check_mid("gemm_mid_silu_bf16", X, W, M, two_i, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(two_i % 2 == 0, "gemm_mid_silu_bf16: gate and up rows must be equally many");
  const int kper = (K + BK - 1) / BK * BK;
  const dim3 grid(pyre_gemm_mid_silu_blocks(M, two_i), 1);
  const bf16* x = static_cast<const bf16*>(X);
  const bf16* w = static_cast<const bf16*>(W);
  if (M > 192) {
    hipLaunchKernelGGL((gemm_mid_kernel<2, 4, 2, kSiluMul, 8, 3>), grid, dim3(64 * 16), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M > 128) {
    hipLaunchKernelGGL((gemm_mid_kernel<2, 3, 2, kSiluMul, 8, 3>), grid, dim3(64 * 14), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 32 && silu_features(M, two_i) == 128) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 1, 4, kSiluMul, 8, 4>), grid, dim3(64 * 12), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 64 && silu_features(M, two_i) == 128) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 2, 4, kSiluMul, 8, 3>), grid, dim3(64 * 16), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 32 && silu_features(M, two_i) == 96) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 1, 3, kSiluMul, 8, 5>), grid, dim3(64 * 11), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 32) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 1, 2, kSiluMul, 8, 6>), grid, dim3(64 * 10), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 64 && silu_features(M, two_i) == 96) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 2, 3, kSiluMul, 8, 4>), grid, dim3(64 * 14), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 64) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 2, 2, kSiluMul, 8, 5>), grid, dim3(64 * 12), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (M <= 96 && silu_features(M, two_i) == 96) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 3, 3, kSiluMul, 6, 4>), grid, dim3(64 * 15), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else if (silu_features(M, two_i) == 96) {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 4, 3, kSiluMul, 4, 3>), grid, dim3(64 * 16), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  } else {
    hipLaunchKernelGGL((gemm_mid_kernel<1, 4, 2, kSiluMul, 8, 4>), grid, dim3(64 * 16), 0, stream, x,
                       static_cast<size_t>(ldx), w, static_cast<size_t>(ldw), out, M, two_i, K, kper);
  }
  return check_launch("gemm_mid_silu_bf16");
}
