// out[m, n] = sum_k X[m, k] W[n, k] for up to 64 rows of X in bfloat16: the matrix
// products of a decode step (pyre/model.py:315-319,338-342), which read every
// weight once and are bound by memory bandwidth. The weights stream from HBM
// straight into MFMA operands, 16 bytes per lane per load; X comes from cache.
//
// The product is computed transposed, out^T = W X^T, so that both operands are
// read along k as they are stored: A = 16 rows of W, B = 16 rows of X, D = a
// 16 (n) x 16 (m) tile with four consecutive n per lane.
//
// A block owns RT tiles of 16 output columns; its four waves split the block's
// k range in interleaved runs of 128 and add their tiles up through LDS in the order 0..3. `ksplit` blocks
// may share a tile (grid.y); each then writes a partial sum that the consumer
// adds in the order 0..ksplit-1, so that the result does not depend on which
// block finishes first.
//
// Epilogues: kPartials stores float32 [ksplit][M][N]; kSiluMul (RT = 2: a tile
// of gate rows and the tile of up rows of the same features, ksplit = 1) stores
// bfloat16 silu(gate) * up, [M][N/2].
#include <type_traits>

#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

enum Epilogue { kPartials = 0, kSiluMul = 1 };
constexpr int kRun = 128;  // k elements a wave takes at a time

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

template <int RT, int MT, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16* __restrict__ X, size_t ldx,
                                                          const bf16* __restrict__ W, size_t ldw,
                                                          void* __restrict__ out, int M, int N, int K,
                                                          int kper) {
  __shared__ f32x4 red[3][RT][MT][64];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int ks = blockIdx.y;
  // Rows of W that this block's tiles cover. For kSiluMul, N counts gate and up
  // rows together: tile 0 = gate rows n0.., tile 1 = up rows N/2 + n0...
  const int half = N / 2;
  int row[RT];
  bool row_ok[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (EPI == kSiluMul) {
      const int n = blockIdx.x * 16 + r;
      row[t] = t * half + n;
      row_ok[t] = n < half;
    } else {
      row[t] = (blockIdx.x * RT + t) * 16 + r;
      row_ok[t] = row[t] < N;
    }
  }
  // The block's k range [kbeg, kend) goes to its waves in runs of 128: wave w takes
  // runs w, w + 4, ... so that the four waves together read 1 KB of each row at a time.
  const int kbeg = ks * kper;
  const int kend = min(K, kbeg + kper);

  f32x4 acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bf16* wp[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) wp[t] = W + static_cast<size_t>(row_ok[t] ? row[t] : 0) * ldw + 8 * g;
  const bf16* xp[MT];
  bool x_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    x_ok[mt] = 16 * mt + r < M;
    xp[mt] = X + static_cast<size_t>(x_ok[mt] ? 16 * mt + r : 0) * ldx + 8 * g;
  }

  for (int kr = kbeg + wave * kRun; kr < kend; kr += 4 * kRun) {
    bf16x8 a[kRun / 32][RT], b[kRun / 32][MT];
#pragma unroll
    for (int u = 0; u < kRun / 32; ++u) {
      const int k0 = kr + 32 * u;
      const bool k_ok = k0 + 8 * g < kend;  // K is a multiple of 8: a lane's 8 elements are in or out together
#pragma unroll
      for (int t = 0; t < RT; ++t) a[u][t] = (k_ok && row_ok[t]) ? ld128(wp[t] + k0) : zero128();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = (k_ok && x_ok[mt]) ? ld128(xp[mt] + k0) : zero128();
    }
#pragma unroll
    for (int u = 0; u < kRun / 32; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], b[u][mt], acc[t][mt], 0, 0, 0);
  }

  // Waves 1..3 hand their tiles to wave 0, which adds them in a fixed order.
  if (wave > 0) {
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) red[wave - 1][t][mt][lane] = acc[t][mt];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int w = 0; w < 3; ++w)
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[t][mt] += red[w][t][mt][lane];

  // Lane holds out^T[n = tile row 4g + j][m = 16 mt + r].
  if (EPI == kPartials) {
    float* o = static_cast<float*>(out) + static_cast<size_t>(ks) * M * N;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int n = (blockIdx.x * RT + t) * 16 + 4 * g;
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
    const int n = blockIdx.x * 16 + 4 * g;
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

// ---------------------------------------------------------------------------
// Second form, for more rows of X: the four waves of a block take different
// output tiles over the same k range, and X goes through LDS once per block
// (double-buffered runs of 128 k) instead of once per wave from cache. W is
// prefetched one run ahead into registers.
// ---------------------------------------------------------------------------
constexpr int kPad = 8;  // bf16 elements of padding per LDS row: rows land on different banks

template <int RT, int MT, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_lds_kernel(const bf16* __restrict__ X, size_t ldx,
                                                              const bf16* __restrict__ W, size_t ldw,
                                                              void* __restrict__ out, int M, int N, int K,
                                                              int kper) {
  __shared__ __attribute__((aligned(16))) bf16 xs[2][MT * 16][kRun + kPad];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, r = lane & 15, g = lane >> 4;
  const int ks = blockIdx.y;
  const int half = N / 2;
  const int tile0 = (blockIdx.x * 4 + wave) * (EPI == kSiluMul ? 1 : RT);
  int row[RT];
  bool row_ok[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    if (EPI == kSiluMul) {
      const int n = tile0 * 16 + r;
      row[t] = t * half + n;
      row_ok[t] = n < half;
    } else {
      row[t] = (tile0 + t) * 16 + r;
      row_ok[t] = row[t] < N;
    }
  }
  const int kbeg = ks * kper, kend = min(K, kbeg + kper);
  const int nruns = (kend - kbeg + kRun - 1) / kRun;

  f32x4 acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};

  const bf16* wp[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) wp[t] = W + static_cast<size_t>(row_ok[t] ? row[t] : 0) * ldw + 8 * g;

  // X staging: 16-byte pieces, MT per thread per run: piece p -> (row p / 16, k 8 * (p % 16)).
  auto load_x = [&](int kr, bf16x8 (&xr)[MT]) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int p = threadIdx.x + 256 * i, xrow = p / (kRun / 8), k = kr + 8 * (p % (kRun / 8));
      xr[i] = (xrow < M && k < kend) ? ld128(X + static_cast<size_t>(xrow) * ldx + k) : zero128();
    }
  };
  auto store_x = [&](int stage, const bf16x8 (&xr)[MT]) {
#pragma unroll
    for (int i = 0; i < MT; ++i) {
      const int p = threadIdx.x + 256 * i;
      *reinterpret_cast<bf16x8*>(&xs[stage][p / (kRun / 8)][8 * (p % (kRun / 8))]) = xr[i];
    }
  };
  auto load_w = [&](int kr, bf16x8 (&a)[kRun / 32][RT]) {
#pragma unroll
    for (int u = 0; u < kRun / 32; ++u) {
      const int k0 = kr + 32 * u;
      const bool k_ok = k0 + 8 * g < kend;
#pragma unroll
      for (int t = 0; t < RT; ++t) a[u][t] = (k_ok && row_ok[t]) ? ld128(wp[t] + k0) : zero128();
    }
  };

  bf16x8 xr[MT], a[kRun / 32][RT], an[kRun / 32][RT];
  if (nruns > 0) {
    load_x(kbeg, xr);
    load_w(kbeg, a);
    store_x(0, xr);
  }
  for (int c = 0; c < nruns; ++c) {
    __syncthreads();  // run c is in xs[c & 1]; everyone is done reading xs[(c + 1) & 1]
    const bool more = c + 1 < nruns;
    if (more) {
      load_x(kbeg + (c + 1) * kRun, xr);
      load_w(kbeg + (c + 1) * kRun, an);
    }
#pragma unroll
    for (int u = 0; u < kRun / 32; ++u) {
      bf16x8 b[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        b[mt] = *reinterpret_cast<const bf16x8*>(&xs[c & 1][16 * mt + r][32 * u + 8 * g]);
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], b[mt], acc[t][mt], 0, 0, 0);
    }
    if (more) {
      store_x((c + 1) & 1, xr);
#pragma unroll
      for (int u = 0; u < kRun / 32; ++u)
#pragma unroll
        for (int t = 0; t < RT; ++t) a[u][t] = an[u][t];
    }
  }

  if (EPI == kPartials) {
    float* o = static_cast<float*>(out) + static_cast<size_t>(ks) * M * N;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const int n = (tile0 + t) * 16 + 4 * g;
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
    const int n = tile0 * 16 + 4 * g;
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
int launch_lds(int mt, dim3 grid, hipStream_t stream, const bf16* X, size_t ldx, const bf16* W, size_t ldw,
               void* out, int M, int N, int K, int kper) {
#define PYRE_LAUNCH_MT(MTV)                                                                              \
  hipLaunchKernelGGL((gemm_skinny_lds_kernel<RT, MTV, EPI>), grid, dim3(256), 0, stream, X, ldx, W, ldw, \
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

// ---------------------------------------------------------------------------
// Third form: W, too, goes through LDS. A block owns 64 * RT consecutive rows of W
// (for kSiluMul: 64 gate rows and the 64 up rows of the same features). Its threads
// load each run of 128 k with 16 consecutive threads on 256 contiguous bytes of one
// row, so that the memory system sees whole cache lines instead of the 64-byte
// pieces of the MFMA operand layout; the waves then read their operands from LDS.
// The next run's global loads are in flight while the current run is multiplied.
// ---------------------------------------------------------------------------
template <int RT, int MT, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_staged_kernel(const bf16* __restrict__ X, size_t ldx,
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
int launch_staged(int mt, dim3 grid, hipStream_t stream, const bf16* X, size_t ldx, const bf16* W, size_t ldw,
                  void* out, int M, int N, int K, int kper) {
#define PYRE_LAUNCH_MT(MTV)                                                                                 \
  hipLaunchKernelGGL((gemm_skinny_staged_kernel<RT, MTV, EPI>), grid, dim3(256), 0, stream, X, ldx, W, ldw, \
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

template <int RT, int EPI>
int launch(int mt, dim3 grid, hipStream_t stream, const bf16* X, size_t ldx, const bf16* W, size_t ldw,
           void* out, int M, int N, int K, int kper) {
#define PYRE_LAUNCH_MT(MTV)                                                                          \
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

// out: float32 [ksplit][M][N]. The block's k range is split over its four waves.
extern "C" int pyre_gemm_skinny_bf16(const void* X, long ldx, const void* W, long ldw, float* out,
                                     int M, int N, int K, int ksplit, int form, hipStream_t stream) {
  if (int rc = check_common("gemm_skinny_bf16", M, N, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(ksplit >= 1 && ksplit <= 64, "gemm_skinny_bf16: ksplit=%d", ksplit);
  const int mt = (M + 15) / 16;
  const int tiles = (N + 15) / 16;
  if ((form & 15) == 2) {  // W and X through LDS
    const int rt = tiles >= 2048 ? 2 : 1;
    const int kper = ((K + ksplit - 1) / ksplit + kRun - 1) / kRun * kRun;
    const dim3 grid((tiles + 4 * rt - 1) / (4 * rt), ksplit);
    const bf16* x = static_cast<const bf16*>(X);
    const bf16* w = static_cast<const bf16*>(W);
    int rc = rt == 2 ? launch_staged<2, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper)
                     : launch_staged<1, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper);
    PYRE_REQUIRE(rc == 0, "gemm_skinny_bf16: no kernel for %d rows", M);
    return check_launch("gemm_skinny_bf16");
  }
  if ((form & 15) == 1) {  // waves on different tiles, X through LDS
    const int rt = tiles >= 2048 ? 2 : 1;
    const int kper = ((K + ksplit - 1) / ksplit + kRun - 1) / kRun * kRun;
    const dim3 grid((tiles + 4 * rt - 1) / (4 * rt), ksplit);
    const bf16* x = static_cast<const bf16*>(X);
    const bf16* w = static_cast<const bf16*>(W);
    int rc = rt == 2 ? launch_lds<2, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper)
                     : launch_lds<1, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper);
    PYRE_REQUIRE(rc == 0, "gemm_skinny_bf16: no kernel for %d rows", M);
    return check_launch("gemm_skinny_bf16");
  }
  // Form 0: tiles per block. More tiles per block mean fewer reads of X (each block
  // reads all of X's k range once) but fewer blocks; `form` may carry a choice in
  // its upper bits (form = 0 + 16 * tiles), else it is made from the sizes.
  int rt = form >> 4;
  if (rt == 0) rt = tiles >= 4096 ? 2 : 1;  // measured: more tiles per block only pay for very wide products
  // k per block, a multiple of what its four waves take in one round
  const int kper = ((K + ksplit - 1) / ksplit + 4 * kRun - 1) / (4 * kRun) * (4 * kRun);
  const dim3 grid((tiles + rt - 1) / rt, ksplit);
  const bf16* x = static_cast<const bf16*>(X);
  const bf16* w = static_cast<const bf16*>(W);
  int rc = 1;
  if (rt == 4) rc = launch<4, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper);
  else if (rt == 2) rc = launch<2, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper);
  else if (rt == 1) rc = launch<1, kPartials>(mt, grid, stream, x, ldx, w, ldw, out, M, N, K, kper);
  PYRE_REQUIRE(rc == 0, "gemm_skinny_bf16: no kernel for %d rows, %d tiles per block", M, rt);
  return check_launch("gemm_skinny_bf16");
}

// W = [gate rows; up rows] (2I x K); out: bfloat16 [M][I] = silu(X gate^T) * (X up^T).
extern "C" int pyre_gemm_skinny_silu_bf16(const void* X, long ldx, const void* W, long ldw, void* out,
                                          int M, int two_i, int K, int form, hipStream_t stream) {
  if (int rc = check_common("gemm_skinny_silu_bf16", M, two_i, K, ldx, ldw)) return rc;
  PYRE_REQUIRE(two_i % 2 == 0, "gemm_skinny_silu_bf16: gate and up rows must be equally many");
  const int mt = (M + 15) / 16;
  if (form == 2) {
    const int kper = (K + kRun - 1) / kRun * kRun;
    const dim3 grid(((two_i / 2 + 15) / 16 + 3) / 4, 1);
    int rc = launch_staged<2, kSiluMul>(mt, grid, stream, static_cast<const bf16*>(X), ldx,
                                        static_cast<const bf16*>(W), ldw, out, M, two_i, K, kper);
    PYRE_REQUIRE(rc == 0, "gemm_skinny_silu_bf16: no kernel for %d rows", M);
    return check_launch("gemm_skinny_silu_bf16");
  }
  if (form == 1) {
    const int kper = (K + kRun - 1) / kRun * kRun;
    const dim3 grid(((two_i / 2 + 15) / 16 + 3) / 4, 1);
    int rc = launch_lds<2, kSiluMul>(mt, grid, stream, static_cast<const bf16*>(X), ldx,
                                     static_cast<const bf16*>(W), ldw, out, M, two_i, K, kper);
    PYRE_REQUIRE(rc == 0, "gemm_skinny_silu_bf16: no kernel for %d rows", M);
    return check_launch("gemm_skinny_silu_bf16");
  }
  const int kper = (K + 4 * kRun - 1) / (4 * kRun) * (4 * kRun);
  const dim3 grid((two_i / 2 + 15) / 16, 1);
  int rc = launch<2, kSiluMul>(mt, grid, stream, static_cast<const bf16*>(X), ldx,
                               static_cast<const bf16*>(W), ldw, out, M, two_i, K, kper);
  PYRE_REQUIRE(rc == 0, "gemm_skinny_silu_bf16: no kernel for %d rows", M);
  return check_launch("gemm_skinny_silu_bf16");
}
