// out[m, n] = sum_k X[m, k] W[n, k] for up to 64 rows of X in bfloat16: the matrix
// products of a decode step (pyre/model.py:315-319,338-342), which read every
// weight once and are bound by memory bandwidth.
//
// The product is computed transposed, out^T = W X^T, so that both operands are
// read along k as they are stored: A = 16 rows of W, B = 16 rows of X, D = a
// 16 (n) x 16 (m) tile with four consecutive n per lane (MFMA 16x16x32).
//
// A block owns 64 RT consecutive rows of W and walks its k range in runs of 128. Its
// threads load a run with 16 consecutive threads on 256 contiguous bytes of one row, so
// that the memory system sees whole cache lines, not the 64-byte pieces of the MFMA
// operand layout; W and X go through LDS, and the four waves, each on RT tiles of 16
// rows, read their operands there. The next run's loads are in flight while the current
// run is multiplied. `ksplit` blocks may share rows (grid.y); each then writes a
// partial sum that the consumer adds in the order 0..ksplit-1, so that the result does
// not depend on which block finishes first.
//
// Epilogues: kPartials stores float32 [ksplit][M][N]; kSiluMul (RT = 2: 64 gate rows
// and the 64 up rows of the same features, ksplit = 1) stores bfloat16
// silu(gate) * up, [M][N/2].
#include <type_traits>

#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum Epilogue { kPartials = 0, kSiluMul = 1 };
constexpr int kRun = 128;  // k elements a block takes at a time

__device__ inline bf16x8 ld128(const bf16* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}
// Weights are read once per step: a non-temporal load keeps them from displacing what
// the caches hold and streams measurably faster from HBM.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ inline bf16x8 ld128_stream(const bf16* p) {
  return __builtin_bit_cast(bf16x8, __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p)));
}
__device__ inline bf16x8 zero128() {
  uint4 z = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, z);
}
__device__ inline uint32_t pack2(float lo, float hi) { return pack_bf16x2(lo, hi); }

constexpr int kPad = 8;  // bf16 elements of padding per LDS row: rows land on different banks

template <int RT, int MT, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16* __restrict__ X, size_t ldx,
                                                                 const bf16* __restrict__ W, size_t ldw,
                                                                 void* __restrict__ out, int M, int N, int K,
                                                                 int kper) {
  constexpr int R = 64 * RT;               // rows of W per block
  constexpr int WP = R * (kRun / 8) / 256;  // 16-byte pieces of W per thread and run
  __shared__ __attribute__((aligned(16))) bf16 wl[R][kRun + kPad];
  __shared__ __attribute__((aligned(16))) bf16 xl[MT * 16][kRun + kPad];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, r = lane & 15, g = lane >> 4;
  const int ks = blockIdx.y;
  const int half = N / 2;
  const int kbeg = ks * kper, kend = min(K, kbeg + kper);
  const int nruns = (kend - kbeg + kRun - 1) / kRun;

  // Global row of LDS row `lr`, or -1 past the end.
  auto global_row = [&](int lr) {
    if (EPI == kSiluMul) {
      const int f = blockIdx.x * 64 + (lr & 63);
      return f < half ? (lr >> 6) * half + f : -1;
    }
    const int n = blockIdx.x * R + lr;
    return n < N ? n : -1;
  };
  const bf16* wsrc[WP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    const int p = tid + 256 * i, gr = global_row(p / (kRun / 8));
    wsrc[i] = gr < 0 ? nullptr : W + static_cast<size_t>(gr) * ldw + 8 * (p % (kRun / 8));
  }
  auto fetch = [&](int kr, bf16x8 (&wr)[WP], bf16x8 (&xr)[MT]) {
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int k = kr + 8 * ((tid + 256 * i) % (kRun / 8));
      wr[i] = (wsrc[i] && k < kend) ? ld128_stream(wsrc[i] + kr) : zero128();
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int p = tid + 256 * i, xrow = p / (kRun / 8), k = kr + 8 * (p % (kRun / 8));
      xr[i] = (xrow < M && k < kend) ? ld128(X + static_cast<size_t>(xrow) * ldx + k) : zero128();
    }
  };
  auto stash = [&](const bf16x8 (&wr)[WP], const bf16x8 (&xr)[MT]) {
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + 256 * i;
      *reinterpret_cast<bf16x8*>(&wl[p / (kRun / 8)][8 * (p % (kRun / 8))]) = wr[i];
    }
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int p = tid + 256 * i;
      *reinterpret_cast<bf16x8*>(&xl[p / (kRun / 8)][8 * (p % (kRun / 8))]) = xr[i];
    }
  };

  f32x4 acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  // LDS rows of this wave's tiles.
  int lrow[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) lrow[t] = (EPI == kSiluMul ? t * 64 + wave * 16 : (wave * RT + t) * 16) + r;

  bf16x8 wr[WP], xr[MT];
  if (nruns > 0) fetch(kbeg, wr, xr);
  for (int c = 0; c < nruns; ++c) {
    stash(wr, xr);
    __syncthreads();
    if (c + 1 < nruns) fetch(kbeg + (c + 1) * kRun, wr, xr);
#pragma unroll
    for (int u = 0; u < kRun / 32; ++u) {
      bf16x8 a[RT], b[MT];
#pragma unroll
      for (int t = 0; t < RT; ++t) a[t] = *reinterpret_cast<const bf16x8*>(&wl[lrow[t]][32 * u + 8 * g]);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[mt] = *reinterpret_cast<const bf16x8*>(&xl[16 * mt + r][32 * u + 8 * g]);
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t], b[mt], acc[t][mt], 0, 0, 0);
    }
    __syncthreads();  // everyone is done with this run before the next one overwrites it
  }

  if (EPI == kPartials) {
    float* o = static_cast<float*>(out) + static_cast<size_t>(ks) * M * N;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int n = blockIdx.x * R + (wave * RT + t) * 16 + 4 * g;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = 16 * mt + r;
        if (m >= M || n >= N) continue;
        float* dst = o + static_cast<size_t>(m) * N + n;
        if (n + 3 < N && (N & 3) == 0) {
          *reinterpret_cast<f32x4*>(dst) = acc[t][mt];
        } else {
          for (int j = 0; j < 4 && n + j < N; ++j) dst[j] = acc[t][mt][j];
        }
      }
    }
  } else {
    bf16* o = static_cast<bf16*>(out);
    const int n = blockIdx.x * 64 + wave * 16 + 4 * g;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = 16 * mt + r;
      if (m >= M || n >= half) continue;
      float y[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float gate = acc[0][mt][j], up = acc[RT - 1][mt][j];
        y[j] = gate / (1.f + __expf(-gate)) * up;
      }
      bf16* dst = o + static_cast<size_t>(m) * half + n;
      if (n + 3 < half && (half & 3) == 0) {
        *reinterpret_cast<uint2*>(dst) = uint2{pack2(y[0], y[1]), pack2(y[2], y[3])};
      } else {
        for (int j = 0; j < 4 && n + j < half; ++j) dst[j] = from_float<bf16>(y[j]);
      }
    }
  }
}

template <int RT, int EPI>
int launch_skinny(int mt, dim3 grid, hipStream_t stream, const bf16* X, size_t ldx, const bf16* W, size_t ldw,
                  void* out, int M, int N, int K, int kper) {
#define PYRE_LAUNCH_MT(MTV)                                                                                 \
  hipLaunchKernelGGL((gemm_skinny_kernel<RT, MTV, EPI>), grid, dim3(256), 0, stream, X, ldx, W, ldw, \
                     out, M, N, K, kper)
  switch (mt) {
    case 1: PYRE_LAUNCH_MT(1); return 0;
    case 2: PYRE_LAUNCH_MT(2); return 0;
    case 3: PYRE_LAUNCH_MT(3); return 0;
    case 4: PYRE_LAUNCH_MT(4); return 0;
  }
#undef PYRE_LAUNCH_MT
  return 1;
}

int check_common(const char* who, int M, int N, int K, long ldx, long ldw) {
  PYRE_REQUIRE(M >= 1 && M <= 64, "%s: %d rows; this kernel takes 1..64", who, M);
  PYRE_REQUIRE(N >= 1 && K >= 8 && K % 8 == 0, "%s: K=%d must be a positive multiple of 8 (N=%d)", who, K, N);
  PYRE_REQUIRE(ldx >= K && ldx % 8 == 0 && ldw >= K && ldw % 8 == 0,
               "%s: row strides must be multiples of 8 elements and at least K", who);
  return 0;
}

}  // namespace

extern "C" int pyre_gemm_skinny_supports(int M, int N, int K, long ldx, long ldw) {
  return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && ldx >= K && ldx % 8 == 0 && ldw >= K &&
         ldw % 8 == 0;
}

// out: float32 [ksplit][M][N].
extern "C" int pyre_gemm_skinny_bf16(const void* X, long ldx, const void* W, long ldw, float* out,
                                     int M, int N, int K, int ksplit, hipStream_t stream) {
  if (int rc = check_common("gemm_skinny_bf16", M, N, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(ksplit >= 1 && ksplit <= 64, "gemm_skinny_bf16: ksplit=%d", ksplit);
  const int mt = (M + 15) / 16;
  const int tiles = (N + 15) / 16;
  const int rt = tiles >= 2048 ? 2 : 1;  // wide products: 128 rows per block
  const int kper = ((K + ksplit - 1) / ksplit + kRun - 1) / kRun * kRun;
  const dim3 grid((tiles + 4 * rt - 1) / (4 * rt), ksplit);
  const bf16* x = static_cast<const bf16*>(X);
  const bf16* w = static_cast<const bf16*>(W);
  const int rc = rt == 2 ? launch_skinny<2, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper)
                         : launch_skinny<1, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper);
  PYRE_REQUIRE(rc == 0, "gemm_skinny_bf16: no kernel for %d rows", M);
  return check_launch("gemm_skinny_bf16");
}

// W = [gate rows; up rows] (2I x K); out: bfloat16 [M][I] = silu(X gate^T) * (X up^T).
extern "C" int pyre_gemm_skinny_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out,
                                          int M, int two_i, int K, hipStream_t stream) {
  if (int rc = check_common("gemm_skinny_silu_bf16", M, two_i, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(two_i % 2 == 0, "gemm_skinny_silu_bf16: gate and up rows must be equally many");
  const int mt = (M + 15) / 16;
  const int kper = (K + kRun - 1) / kRun * kRun;
  const dim3 grid(((two_i / 2 + 15) / 16 + 3) / 4, 1);
  const int rc = launch_skinny<2, kSiluMul>(mt, grid, stream, static_cast<const bf16*>(X), ldx,
                                            static_cast<const bf16*>(W), ldw, out, M, two_i, K, kper);
  PYRE_REQUIRE(rc == 0, "gemm_skinny_silu_bf16: no kernel for %d rows", M);
  return check_launch("gemm_skinny_silu_bf16");
}
