// out[m, n] = sum_k A[m, k] * W[n, k] (+ bias[n]) with all three in float32, on the matrix
// cores' true 32-bit instruction (v_mfma_f32_32x32x2_f32: float32 operands, float32 products
// and sums; no reduced-precision mode is involved). This is the product of the 32-bit path
// of the model (`pyre/model.py:92-94,125,139,201` are the products it stands for); operands
// of mixed element types stay with gemm_generic.hip.
//
// As in the weight-streaming kernels the product is computed transposed, out^T = W A^T: the
// 32 rows of an MFMA tile are output columns n, its 32 columns are rows m, so that a lane
// holds runs of four consecutive n of one row m and stores them as one float4.
//
// The instruction adds an element's products one after the other, each with one fused
// multiply-add, in the order of its k (for 32x32x2: lanes 0..31, then lanes 32..63; for 16x16x4:
// the four groups of 16 lanes in turn), exactly as a chain of fmaf() does. k is walked in stages
// of 16 through LDS, and within a stage in the order 0, 4, 8, 12, 1, 5, 9, 13, 2, ..., 15: step s
// (0..7) of 32x32x2 multiplies k = 8 (s & 1) + (s >> 1) in lanes 0..31 and that k + 4 in lanes
// 32..63, so that a lane reads its eight values of a stage as two 16-byte LDS loads (pieces
// `half` and `half` + 2); step i (0..3) of 16x16x4 multiplies k = 4 g + i in its lane group g (one
// 16-byte load). The order in which an element's products are added is a function of k alone and
// the same for every tile shape and both instructions below, so an element's value does not depend
// on the shape, on the number of rows in the step or on where the row lies in it, bit for bit.
//
// k may be split into `ksplit` parts (grid.z), each writing a partial sum out[s] that the
// consumer adds in the order 0..ksplit-1: products with few output columns and a long k would
// otherwise leave most of the chip idle. The caller chooses ksplit from N and K alone.
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int BK = 16;      // k per stage
constexpr int LD = BK + 4;  // floats per LDS row: 80 bytes, so that eight rows' 16-byte pieces fall on distinct banks

// Four consecutive k of one row; zero where the row or the k is not there.
__device__ inline f32x4 load_k4(const float* base, size_t ld, int row, int rows, int k, int K, bool vec_ok) {
  if (row >= rows || k >= K) return f32x4{0.f, 0.f, 0.f, 0.f};
  const float* p = base + static_cast<size_t>(row) * ld + k;
  if (vec_ok && k + 3 < K) return *reinterpret_cast<const f32x4*>(p);
  f32x4 v = {0.f, 0.f, 0.f, 0.f};
  for (int j = 0; j < 4 && k + j < K; ++j) v[j] = p[j];
  return v;
}

// WN x WM waves (along n and along m), each on TN x TM tiles of 32 x 32.
template <int WN, int WM, int TN, int TM>
__global__ __launch_bounds__(64 * WN * WM) void gemm_f32_mfma_kernel(
    const float* __restrict__ A, size_t lda, const float* __restrict__ W, size_t ldw,
    const void* __restrict__ bias, int bias_dt, float* __restrict__ out, size_t ldo, size_t part_stride, int M,
    int N, int K, int kper, int vec_ok) {
  constexpr int NT = 64 * WN * WM, BN = WN * TN * 32, BM = WM * TM * 32;
  constexpr int WP = (BN * 4 + NT - 1) / NT, AP = (BM * 4 + NT - 1) / NT;  // 16-byte pieces per thread and stage
  __shared__ __attribute__((aligned(16))) float Ws[BN][LD];
  __shared__ __attribute__((aligned(16))) float As[BM][LD];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, half = lane >> 5, c = lane & 31;
  const int wn = wave % WN, wm = wave / WN;
  const int n0 = blockIdx.x * BN, m0 = blockIdx.y * BM;
  const int kbeg = blockIdx.z * kper;
  K = min(K, kbeg + kper);  // this part's end
  out += blockIdx.z * part_stride;
  if (blockIdx.z) bias = nullptr;  // the bias belongs to one part only

  f32x4 wr[WP], ar[AP];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + NT * i;
      wr[i] = p < BN * 4 ? load_k4(W, ldw, n0 + p / 4, N, k0 + 4 * (p % 4), K, vec_ok) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < AP; ++i) {
      const int p = tid + NT * i;
      ar[i] = p < BM * 4 ? load_k4(A, lda, m0 + p / 4, M, k0 + 4 * (p % 4), K, vec_ok) : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < WP; ++i) {
      const int p = tid + NT * i;
      if (p < BN * 4) *reinterpret_cast<f32x4*>(&Ws[p / 4][4 * (p % 4)]) = wr[i];
    }
#pragma unroll
    for (int i = 0; i < AP; ++i) {
      const int p = tid + NT * i;
      if (p < BM * 4) *reinterpret_cast<f32x4*>(&As[p / 4][4 * (p % 4)]) = ar[i];
    }
  };

  f32x16 acc[TN][TM];
#pragma unroll
  for (int t = 0; t < TN; ++t)
#pragma unroll
    for (int u = 0; u < TM; ++u)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[t][u][i] = 0.f;

  fetch(kbeg);
  for (int k0 = kbeg; k0 < K; k0 += BK) {
    stash();
    __syncthreads();
    if (k0 + BK < K) fetch(k0 + BK);  // in flight while this stage is multiplied
    f32x4 a[TN][2], b[TM][2];
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) a[t][h] = *reinterpret_cast<const f32x4*>(&Ws[(wn * TN + t) * 32 + c][4 * half + 8 * h]);
#pragma unroll
    for (int u = 0; u < TM; ++u)
#pragma unroll
      for (int h = 0; h < 2; ++h) b[u][h] = *reinterpret_cast<const f32x4*>(&As[(wm * TM + u) * 32 + c][4 * half + 8 * h]);
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int t = 0; t < TN; ++t)
#pragma unroll
        for (int u = 0; u < TM; ++u)
          acc[t][u] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t][s & 1][s >> 1], b[u][s & 1][s >> 1], acc[t][u], 0, 0, 0);
    __syncthreads();
  }

  // acc[t][u][4 i + j]: output column n = tile row 8 i + 4 half + j, output row m = tile column c.
#pragma unroll
  for (int u = 0; u < TM; ++u) {
    const int m = m0 + (wm * TM + u) * 32 + c;
    if (m >= M) continue;
#pragma unroll
    for (int t = 0; t < TN; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int n = n0 + (wn * TN + t) * 32 + 8 * i + 4 * half;
        if (n >= N) continue;
        float v[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          v[j] = acc[t][u][4 * i + j];
          if (bias && n + j < N) v[j] += load_as_float(bias, bias_dt, n + j);
        }
        float* dst = out + static_cast<size_t>(m) * ldo + n;
        if (n + 3 < N && (ldo & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
          *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
        } else {
          for (int j = 0; j < 4 && n + j < N; ++j) dst[j] = v[j];
        }
      }
  }
}

// The same product for a decode step's rows (M <= 64), as a stream over the weights. A block
// is one wave with 32 output columns, so there is no barrier. It has a ring of R slots in LDS, a
// slot being 32 k (two stages) of its 32 rows of W (4 KB) and of XR rows of A (XR = 8, 16, 32 or 64,
// whichever holds M: 1 to 8 KB), filled by loads that go from memory straight into LDS: while
// slot j is multiplied, slot j + 1 is read from LDS into registers and the R - 2 after it are on
// their way. A load instruction takes whole 128-byte lines (8 rows x 32 k); the 16-byte pieces
// of a row are exchanged among themselves by the row's number so that the matrix instruction's
// operand reads (a lane's row, eight k of a stage) spread over the banks. Stages, steps and
// parts of k are those of the kernel above, and an element of the result depends on its own
// row of A and row of W alone: the sums are the same bit for bit, however many of the
// instruction's 32 columns carry a row. With few rows the chain of dependent instructions of a
// wave, not memory, sets the pace (a slot of 4 KB in about 0.6 us), and with 64 rows the matrix
// cores' float32 rate does; a small ring lets several blocks share a compute unit.
constexpr int kStreamMaxRows = 64;
constexpr int kMaxDevices = 64;
constexpr int kSlotK = 32;

__device__ inline void load_to_lds(const void* src, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(lds_addr) : "memory", "m0");
}
template <int N>
__device__ inline void wait_loads() {
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
__device__ __attribute__((aligned(16))) const unsigned kZeroPiece[4] = {0u, 0u, 0u, 0u};

// NW = 4 (steps of 17 to 64 rows): four such waves, one on each SIMD, share the step's rows: a slot
// holds the four waves' weights and one copy of the rows, of which every wave loads a quarter, and
// a barrier per slot tells a wave that the others' quarters are there. A wave alone reads the rows
// from L2 once per 32 output columns, more bytes than its weights at 64 rows, and has LDS for one
// slot on its way; four waves together have it for four (the ring is dynamic shared memory then).
extern __shared__ __attribute__((aligned(1024))) unsigned char stream_ring[];

template <int R, int XR, int NW>
__global__ __launch_bounds__(64 * NW) void gemm_f32_stream_kernel(
    const float* __restrict__ A, size_t lda, const float* __restrict__ W, size_t ldw,
    const void* __restrict__ bias, int bias_dt, float* __restrict__ out, size_t ldo, size_t part_stride, int M,
    int N, int K, int kper) {
  static_assert(NW == 1 || (NW == 4 && XR >= 32), "four waves share 32 or 64 rows");
  constexpr int XL = XR / 8 / NW;               // this wave's load instructions for a slot's rows of A
  constexpr int MT = XR > 32 ? 2 : 1;           // tiles of 32 rows of A
  constexpr int kSlotBytes = 4096 * NW + XR * 128;
  constexpr int L = 4 + XL;                     // a wave's load instructions per slot
  static_assert(L * (R - 2) <= 63, "the wait counter holds 63 loads");
  __shared__ __attribute__((aligned(1024))) unsigned char own_ring[NW == 1 ? R * kSlotBytes : 16];
  unsigned char* const ring = NW == 1 ? own_ring : stream_ring;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, half = lane >> 5, c = lane & 31;
  const int n0 = (blockIdx.x * NW + wave) * 32;
  const int kbeg = blockIdx.z * kper;
  K = min(K, kbeg + kper);  // this part's end
  out += blockIdx.z * part_stride;
  if (blockIdx.z) bias = nullptr;  // the bias belongs to one part only
  const int slots = (K - kbeg + kSlotK - 1) / kSlotK;

  // This lane's share of a slot's loads: of load i, the piece that lands at row 8 i + lane / 8,
  // place lane % 8, which is piece (place ^ swizzle of the row) of the row's 32 k. Columns past
  // the end read the last one's weights and are not stored; rows of A past M read zeros.
  const int lr = lane >> 3, lp = lane & 7;
  const float* wsrc[4];
  int wk[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 8 * i + lr;
    wk[i] = 4 * (lp ^ ((r >> 1) & 7));
    wsrc[i] = W + static_cast<size_t>(min(n0 + r, N - 1)) * ldw + kbeg + wk[i];
  }
  const float* xsrc[XL];
  int xk[XL];
  bool xrow[XL];
#pragma unroll
  for (int i = 0; i < XL; ++i) {
    const int r = 8 * (NW * i + wave) + lr;  // of the slot's instructions for A, this wave's are wave, NW + wave, ...
    xk[i] = 4 * (lp ^ ((r >> 1) & 7));
    xrow[i] = r < M;
    xsrc[i] = A + static_cast<size_t>(xrow[i] ? r : 0) * lda + kbeg + xk[i];
  }
  const unsigned mine = __builtin_amdgcn_readfirstlane(static_cast<unsigned>(reinterpret_cast<uintptr_t>(ring)));
  const float* zero = reinterpret_cast<const float*>(kZeroPiece);

  int fill = 0;  // ring position of the next slot to load
  auto issue = [&](int j) {
    const unsigned dst = mine + fill * kSlotBytes;
    fill = fill + 1 == R ? 0 : fill + 1;
    const int k0 = kSlotK * j, left = j < slots ? K - kbeg - k0 : 0;  // k of this part from the slot's start on
#pragma unroll
    for (int i = 0; i < 4; ++i) load_to_lds(wk[i] < left ? wsrc[i] + k0 : zero, dst + 4096 * wave + 1024 * i);
#pragma unroll
    for (int i = 0; i < XL; ++i)
      load_to_lds(xrow[i] && xk[i] < left ? xsrc[i] + k0 : zero, dst + 4096 * NW + 1024 * (NW * i + wave));
  };
  // The slot that this wave's loads have just filled is whole when the other waves' are there too.
  auto slot_whole = [&]() {
    if (NW > 1) {
      asm volatile("s_waitcnt lgkmcnt(0)" : : : "memory");  // and what this wave read of the slot that is filled next
      __syncthreads();
    }
  };

  if constexpr (XR <= 16) {
    // Sixteen rows or fewer: 16x16x4, whose 16 columns hold the step's rows and whose 16 rows are
    // output columns, two tiles of them a wave. It takes a weight once for 16 rows where 32x32x2
    // takes it once for 32, so that a wave gets through its weights in half the time.
    const int g = lane >> 4, c16 = lane & 15;
    f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
    const int xr = XR == 8 ? c16 & 7 : c16;  // eight rows: the instruction's columns 8..15 read them again and are not stored
    const unsigned char* wpiece0 = ring + c16 * 128;
    const unsigned char* wpiece1 = ring + (16 + c16) * 128;
    const unsigned char* xpiece = ring + 4096 + xr * 128;
    const int swz = (c16 >> 1) & 7, xswz = (xr >> 1) & 7;  // rows c16 and 16 + c16 exchange their pieces alike
    int at = 0;
    auto read = [&](f32x4 (&a)[2][2], f32x4 (&b)[2]) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int piece = 4 * t + g;
        a[0][t] = *reinterpret_cast<const f32x4*>(wpiece0 + at * kSlotBytes + 16 * (piece ^ swz));
        a[1][t] = *reinterpret_cast<const f32x4*>(wpiece1 + at * kSlotBytes + 16 * (piece ^ swz));
        b[t] = *reinterpret_cast<const f32x4*>(xpiece + at * kSlotBytes + 16 * (piece ^ xswz));
      }
      at = at + 1 == R ? 0 : at + 1;
    };
#pragma unroll
    for (int j = 0; j < R - 1; ++j) issue(j);
    f32x4 a[2][2], b[2], an[2][2], bn[2];
    wait_loads<L * (R - 2)>();
    read(a, b);
    for (int j = 0; j < slots; ++j) {
      issue(j + R - 1);
      wait_loads<L * (R - 2)>();
      read(an, bn);
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        if (kSlotK * j + BK * t >= K - kbeg) break;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int u = 0; u < 2; ++u) acc[u] = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u][t][i], b[t][i], acc[u], 0, 0, 0);
      }
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        a[0][t] = an[0][t];
        a[1][t] = an[1][t];
        b[t] = bn[t];
      }
    }
    wait_loads<0>();
    // acc[u][j]: output column n = 16 u + 4 g + j, output row m = c16.
    if (c16 >= M || c16 >= XR) return;
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int n = n0 + 16 * u + 4 * g;
      if (n >= N) continue;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = acc[u][j];
        if (bias && n + j < N) v[j] += load_as_float(bias, bias_dt, n + j);
      }
      float* dst = out + static_cast<size_t>(c16) * ldo + n;
      if (n + 3 < N && (ldo & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
      } else {
        for (int j = 0; j < 4 && n + j < N; ++j) dst[j] = v[j];
      }
    }
  } else {
  f32x16 acc[MT];
#pragma unroll
  for (int u = 0; u < MT; ++u)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[u][i] = 0.f;
  const unsigned char* wpiece = ring + 4096 * wave + c * 128;
  const unsigned char* xpiece = ring + 4096 * NW + c * 128;
  const int swz = (c >> 1) & 7;  // rows c and 32 + c exchange their pieces alike
  int at = 0;  // ring position of the next slot to read
  auto read = [&](f32x4 (&a)[2][2], f32x4 (&b)[MT][2][2]) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int piece = 4 * t + half + 2 * h;
        a[t][h] = *reinterpret_cast<const f32x4*>(wpiece + at * kSlotBytes + 16 * (piece ^ swz));
#pragma unroll
        for (int u = 0; u < MT; ++u) {
          b[u][t][h] = *reinterpret_cast<const f32x4*>(xpiece + at * kSlotBytes + 4096 * u + 16 * (piece ^ swz));
        }
      }
    at = at + 1 == R ? 0 : at + 1;
  };

  // Slot j + 1 is read from LDS while slot j is multiplied, so of the R slots of the ring one is
  // in registers, one being read and R - 2 on their way.
#pragma unroll
  for (int j = 0; j < R - 1; ++j) issue(j);
  f32x4 a[2][2], b[MT][2][2], an[2][2], bn[MT][2][2];
  wait_loads<L * (R - 2)>();  // loads finish in the order of issue: slot 0 is there
  slot_whole();
  read(a, b);
  for (int j = 0; j < slots; ++j) {
    issue(j + R - 1);            // into the position of slot j - 1, read a turn ago (by every wave: the barrier since)
    wait_loads<L * (R - 2)>();   // slot j + 1 is there
    slot_whole();
    read(an, bn);
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      if (kSlotK * j + BK * t >= K - kbeg) break;  // a part that ends with half a slot
#pragma unroll
      for (int s = 0; s < 8; ++s)
#pragma unroll
        for (int u = 0; u < MT; ++u)
          acc[u] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[t][s & 1][s >> 1], b[u][t][s & 1][s >> 1], acc[u], 0, 0, 0);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        a[t][h] = an[t][h];
#pragma unroll
        for (int u = 0; u < MT; ++u) b[u][t][h] = bn[u][t][h];
      }
  }
  wait_loads<0>();  // the loads past the end

  // acc[u][4 i + j]: output column n = tile row 8 i + 4 half + j, output row m = 32 u + tile column c.
#pragma unroll
  for (int u = 0; u < MT; ++u) {
    const int m = 32 * u + c;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int n = n0 + 8 * i + 4 * half;
      if (n >= N) continue;
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[j] = acc[u][4 * i + j];
        if (bias && n + j < N) v[j] += load_as_float(bias, bias_dt, n + j);
      }
      float* dst = out + static_cast<size_t>(m) * ldo + n;
      if (n + 3 < N && (ldo & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
        *reinterpret_cast<f32x4*>(dst) = f32x4{v[0], v[1], v[2], v[3]};
      } else {
        for (int j = 0; j < 4 && n + j < N; ++j) dst[j] = v[j];
      }
    }
  }
  }
}

}  // namespace

extern "C" int pyre_gemm_f32(const float* A, long lda, const float* W, long ldw, const void* bias, int bias_dt,
                             float* out, long ldo, long part_stride, int M, int N, int K, int ksplit,
                             hipStream_t stream) {
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "gemm_f32: unknown bias dtype");
  PYRE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  PYRE_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_f32: a leading dimension is too small");
  PYRE_REQUIRE(ksplit >= 1 && ksplit <= 64 && (ksplit == 1 || part_stride >= static_cast<long>(M) * ldo),
               "gemm_f32: ksplit=%d, partial sums %ld apart", ksplit, part_stride);
  if (M == 0) return 0;
  const int kper = ((K + ksplit - 1) / ksplit + BK - 1) / BK * BK;
  PYRE_REQUIRE(static_cast<long>(ksplit - 1) * kper < K, "gemm_f32: a part of k would be empty (K=%d, ksplit=%d)", K, ksplit);
  // 16-byte loads along k need rows that start on 16 bytes
  const int vec_ok = lda % 4 == 0 && ldw % 4 == 0 && reinterpret_cast<uintptr_t>(A) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(W) % 16 == 0;
  if (M <= kStreamMaxRows && vec_ok && K % 4 == 0) {  // a decode step's rows: the weights as a stream
    const dim3 grid((N + 31) / 32, 1, ksplit);
#define PYRE_STREAM(R, XR)                                                                                         \
  hipLaunchKernelGGL((gemm_f32_stream_kernel<R, XR, 1>), grid, dim3(64), 0, stream, A, static_cast<size_t>(lda), W, \
                     static_cast<size_t>(ldw), bias, bias_dt, out, static_cast<size_t>(ldo),                       \
                     static_cast<size_t>(part_stride), M, N, K, kper)
// four waves a block, the ring in dynamic shared memory (asked for once per device and kernel)
#define PYRE_STREAM4(R, XR)                                                                                        \
  do {                                                                                                             \
    constexpr int kBytes = (R) * (4096 * 4 + (XR) * 128);                                                          \
    static bool asked[kMaxDevices] = {};                                                                           \
    int dev = 0;                                                                                                   \
    PYRE_REQUIRE(hipGetDevice(&dev) == hipSuccess && dev >= 0 && dev < kMaxDevices, "gemm_f32: no device");         \
    if (!asked[dev]) {                                                                                             \
      PYRE_REQUIRE(hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_f32_stream_kernel<R, XR, 4>),           \
                                       hipFuncAttributeMaxDynamicSharedMemorySize, kBytes) == hipSuccess,          \
                   "gemm_f32: %d bytes of LDS a block are refused", kBytes);                                       \
      asked[dev] = true;                                                                                           \
    }                                                                                                              \
    hipLaunchKernelGGL((gemm_f32_stream_kernel<R, XR, 4>), dim3((N + 127) / 128, 1, ksplit), dim3(256), kBytes,    \
                       stream, A, static_cast<size_t>(lda), W, static_cast<size_t>(ldw), bias, bias_dt, out,       \
                       static_cast<size_t>(ldo), static_cast<size_t>(part_stride), M, N, K, kper);                 \
  } while (0)
    if (M <= 8) PYRE_STREAM(4, 8);
    else if (M <= 16) PYRE_STREAM(4, 16);
    else if (M <= 32 && N >= 128) PYRE_STREAM4(7, 32);
    else if (M <= 32) PYRE_STREAM(4, 32);
    else if (N >= 128) PYRE_STREAM4(6, 64);
    else PYRE_STREAM(3, 64);
#undef PYRE_STREAM
#undef PYRE_STREAM4
  } else if (M <= 32) {  // four waves side by side along n
    const dim3 grid((N + 127) / 128, (M + 31) / 32, ksplit);
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<4, 1, 1, 1>), grid, dim3(256), 0, stream, A, static_cast<size_t>(lda), W,
                       static_cast<size_t>(ldw), bias, bias_dt, out, static_cast<size_t>(ldo),
                       static_cast<size_t>(part_stride), M, N, K, kper, vec_ok);
  } else {
    const dim3 grid((N + 127) / 128, (M + 127) / 128, ksplit);
    PYRE_REQUIRE(grid.y <= 65535, "gemm_f32: M=%d too large for one launch", M);
    hipLaunchKernelGGL((gemm_f32_mfma_kernel<2, 2, 2, 2>), grid, dim3(256), 0, stream, A, static_cast<size_t>(lda), W,
                       static_cast<size_t>(ldw), bias, bias_dt, out, static_cast<size_t>(ldo),
                       static_cast<size_t>(part_stride), M, N, K, kper, vec_ok);
  }
  return check_launch("gemm_f32");
}
