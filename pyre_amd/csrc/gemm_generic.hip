// out[m, n] = sum_k A[m, k] * W[n, k] (+ bias[n]) for any sizes, strides and mix of
// fp32 / bf16 operands, accumulated in fp32 with plain fused multiply-adds in
// ascending k: the true 32-bit matrix product of the engine, and the fallback of
// the 16-bit path for shapes the MFMA kernels refuse (`pyre/model.py:92-94,125,139,201`
// are the products it stands for).
#include "pyre_api.h"
#include "pyre_common.h"

using namespace pyre;

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

template <typename TA, typename TW>
__global__ __launch_bounds__(256) void gemm_generic_kernel(
    const TA* __restrict__ A, size_t lda, const int* __restrict__ a_rows, const TW* __restrict__ W,
    size_t ldw, const void* __restrict__ bias, int bias_dt, void* __restrict__ out, int out_dt,
    size_t ldo, int M, int N, int K) {
  // +1 column of padding keeps the transposed reads of the inner loop off one bank.
  __shared__ float As[BK][BM + 1];
  __shared__ float Ws[BK][BN + 1];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int tx = tid % 16, ty = tid / 16;  // 16 x 16 threads, each a 4 x 4 patch

  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  // Each thread loads 4 elements of the A tile and 4 of the W tile per k-step:
  // element e = tid + 256 * r -> (row e / BK, k e % BK).
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int r = 0; r < (BM * BK) / 256; ++r) {
      const int e = tid + 256 * r, row = e / BK, kk = e % BK;
      const int m = m0 + row, k = k0 + kk;
      float v = 0.f;
      if (m < M && k < K) {
        const size_t src = a_rows ? static_cast<size_t>(a_rows[m]) : static_cast<size_t>(m);
        v = to_float(A[src * lda + k]);
      }
      As[kk][row] = v;
    }
#pragma unroll
    for (int r = 0; r < (BN * BK) / 256; ++r) {
      const int e = tid + 256 * r, row = e / BK, kk = e % BK;
      const int n = n0 + row, k = k0 + kk;
      Ws[kk][row] = (n < N && k < K) ? to_float(W[static_cast<size_t>(n) * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], w[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = As[kk][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) w[j] = Ws[kk][tx * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }

#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += load_as_float(bias, bias_dt, n);
      store_from_float(out, out_dt, static_cast<size_t>(m) * ldo + n, v);
    }
  }
}

}  // namespace

extern "C" int pyre_gemm_generic(const void* A, int a_dt, long lda, const int* a_rows,
                                 const void* W, int w_dt, long ldw, const void* bias, int bias_dt,
                                 void* out, int out_dt, long ldo, int M, int N, int K,
                                 hipStream_t stream) {
  PYRE_REQUIRE(known_dtype(a_dt) && known_dtype(w_dt) && known_dtype(out_dt),
               "gemm_generic: unknown dtype");
  PYRE_REQUIRE(!bias || known_dtype(bias_dt), "gemm_generic: unknown bias dtype");
  PYRE_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_generic: bad sizes M=%d N=%d K=%d", M, N, K);
  PYRE_REQUIRE(lda >= K && ldw >= K && ldo >= N, "gemm_generic: a leading dimension is too small");
  if (M == 0) return 0;
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  PYRE_REQUIRE(grid.y <= 65535, "gemm_generic: M=%d too large for one launch", M);
  PYRE_DISPATCH(a_dt, TA, PYRE_DISPATCH(w_dt, TW,
      hipLaunchKernelGGL((gemm_generic_kernel<TA, TW>), grid, dim3(256), 0, stream,
                         static_cast<const TA*>(A), static_cast<size_t>(lda), a_rows,
                         static_cast<const TW*>(W), static_cast<size_t>(ldw), bias, bias_dt, out,
                         out_dt, static_cast<size_t>(ldo), M, N, K)));
  return check_launch("gemm_generic");
}
