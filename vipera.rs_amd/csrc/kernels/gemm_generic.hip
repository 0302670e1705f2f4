// C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]) with every product and sum in 32-bit FMA.
//
// This is the true 32-bit matrix product of the engine (no matrix-core mode of reduced
// precision) and the fallback for mixed storage types. Each output element is summed by one
// thread over k in ascending order, so its value does not depend on M, on the tile it falls in,
// or on what else is in the batch.
//
// The reference computes every linear layer as dot(row of W, activation) with the bias added
// after the product (crates/vipera-backend-cpu/src/model.rs:623-629, 1005-1031); weights are
// row-major [out, in] (crates/vipera-backend-cpu/src/quant.rs:1-4).
#include "common.h"

namespace {
constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

template <typename TA, typename TW, typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                           const float* __restrict__ bias, TC* __restrict__ C,
                                                           int M, int N, int K, long long lda, long long ldc) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int ty = tid / 16, tx = tid % 16;
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  // each thread stages 4 elements of A and 4 of W per k-tile: row = tid / 4, k = (tid % 4) * 4 + e
  const int lr = tid / 4, lk = (tid % 4) * 4;
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lr, wn = n0 + lr;
      As[lk + e][lr] = (am < M && k < K) ? to_float<TA>(A[(size_t)am * lda + k]) : 0.f;
      Ws[lk + e][lr] = (wn < N && k < K) ? to_float<TW>(W[(size_t)wn * K + k]) : 0.f;
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
      if (bias) v += bias[n];
      TC* dst = C + (size_t)m * ldc + n;
      if (ACCUMULATE)
        *dst = from_float<TC>(to_float<TC>(*dst) + v);
      else
        *dst = from_float<TC>(v);
    }
  }
}

template <typename TA, typename TW, typename TC>
int launch(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, long long lda,
           long long ldc, int accumulate, hipStream_t s) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (accumulate)
    gemm_generic_kernel<TA, TW, TC, true><<<grid, 256, 0, s>>>((const TA*)A, (const TW*)W, bias, (TC*)C, M, N, K, lda, ldc);
  else
    gemm_generic_kernel<TA, TW, TC, false><<<grid, 256, 0, s>>>((const TA*)A, (const TW*)W, bias, (TC*)C, M, N, K, lda, ldc);
  VK_LAUNCH_CHECK();
  return 0;
}
}  // namespace

// dtypes: 0 = float, 1 = bfloat16. lda / ldc are row strides in elements.
extern "C" int vk_gemm_generic(const void* A, int a_dtype, const void* W, int w_dtype, const float* bias, void* C,
                               int c_dtype, int M, int N, int K, long long lda, long long ldc, int accumulate,
                               void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc < N) return VK_BAD_ARGUMENT;
  if ((M + BM - 1) / BM > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (key) {
    case 0: return launch<float, float, float>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 1: return launch<float, float, bf16_t>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 2: return launch<float, bf16_t, float>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 3: return launch<float, bf16_t, bf16_t>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 4: return launch<bf16_t, float, float>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 5: return launch<bf16_t, float, bf16_t>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 6: return launch<bf16_t, bf16_t, float>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
    case 7: return launch<bf16_t, bf16_t, bf16_t>(A, W, bias, C, M, N, K, lda, ldc, accumulate, s);
  }
  return VK_BAD_ARGUMENT;
}
