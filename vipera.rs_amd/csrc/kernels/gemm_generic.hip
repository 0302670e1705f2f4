// C[M,N] = A[M,K] * W[N,K]^T (+ bias[N]) with every product and sum in 32-bit FMA.
//
// This is the true 32-bit matrix product of the engine (no matrix-core mode of reduced
// precision) and the fallback for mixed storage types.
//
// The reference computes every linear layer as dot(row of W, activation) with the bias added
// after the product (crates/vipera-backend-cpu/src/model.rs:623-629, 1005-1031); weights are
// row-major [out, in] (crates/vipera-backend-cpu/src/quant.rs:1-4).
//
// One order of summation for every output element, whatever kernel computes it, whatever M is and
// whatever else is in the batch, so that a token's result is the same bit for bit however a step is
// cut or batched:
//   * K is cut into ranges of RANGE_K = 256 consecutive k; a range's sum is one chain
//     acc = fma(a[k], w[k], acc) over ascending k, started at +0;
//   * SLAB_RANGES = 4 consecutive ranges form a slab, whose sum is +0 + r0 + r1 + r2 + r3 in that
//     order (ranges past the end of K count as +0, which changes nothing: a chain that starts at +0
//     never ends at -0);
//   * the element is +0 + s0 + s1 + ... over its slabs in ascending order, then + bias, then,
//     when accumulating, old + that.
// Three kernels follow it. gemm_stream_kernel, for up to 64 rows of A in 32-bit operands, is a stream
// of the weights: the product of a few tokens is bound by the bytes of W. gemm_generic_kernel is a
// plain tiled product for everything else, gemm_generic_wide_kernel its twin with larger tiles for
// 128 rows of A and more.
#include "common.h"

namespace {
constexpr int RANGE_K = 256, SLAB_RANGES = 4, SLAB_K = RANGE_K * SLAB_RANGES;
typedef float f32x4_t __attribute__((ext_vector_type(4)));

// ---------------------------------------------------------------------------------------------
// The tiled product: any operand types, any M. A thread owns a 4 x 4 block of outputs and walks K in
// steps of 16 through LDS; the three levels of sums above are three sets of accumulators.
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
  float acc[TM][TN], slab[TM][TN], total[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = slab[i][j] = total[i][j] = 0.f;

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
    const int done = k0 + BK;  // a multiple of 16, as the range and slab lengths are
    if (done % RANGE_K == 0 || done >= K) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          slab[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    if (done % SLAB_K == 0 || done >= K) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          total[i][j] += slab[i][j];
          slab[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n >= N) continue;
      float v = total[i][j];
      if (bias) v += bias[n];
      TC* dst = C + (size_t)m * ldc + n;
      if (ACCUMULATE)
        *dst = from_float<TC>(to_float<TC>(*dst) + v);
      else
        *dst = from_float<TC>(v);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The same product for 128 rows of A and more (prompts): a 128 x 128 tile, a thread owns 8 x 8 outputs (rows
// 4 ty .. + 3 and 64 + 4 ty .. + 3, columns likewise with tx), so that a step of k costs four 16-byte LDS reads for
// 64 FMAs where the 4 x 4 block above pays two for 16 and is bound by LDS as much as by arithmetic. The next
// 16 k of both operands are on their way from memory into registers while this tile's are multiplied, and go
// into the other half of a double LDS buffer: one barrier per 16 k. Every output element's sums are those of
// the kernel above, in the same order.
constexpr int WIDE = 128, WIDE_ROW = WIDE + 4;

template <typename T>
__device__ __forceinline__ void fetch4(const T* __restrict__ base, long long ld, int row, int rows, int k, int K,
                                       bool vector_ok, float (&dst)[4]) {
  if (row < rows && k + 3 < K && vector_ok) {
    if constexpr (sizeof(T) == 4) {
      const f32x4_t v = *(const f32x4_t*)(base + (size_t)row * ld + k);
#pragma unroll
      for (int e = 0; e < 4; ++e) dst[e] = v[e];
      return;
    }
  }
#pragma unroll
  for (int e = 0; e < 4; ++e) dst[e] = (row < rows && k + e < K) ? to_float<T>(base[(size_t)row * ld + k + e]) : 0.f;
}

template <typename TA, typename TW, typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_generic_wide_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                                const float* __restrict__ bias, TC* __restrict__ C,
                                                                int M, int N, int K, long long lda, long long ldc,
                                                                int a_vector_ok, int w_vector_ok) {
  __shared__ __attribute__((aligned(16))) float As[2][BK][WIDE_ROW];
  __shared__ __attribute__((aligned(16))) float Ws[2][BK][WIDE_ROW];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * WIDE, n0 = blockIdx.x * WIDE;
  const int ty = tid / 16, tx = tid % 16;
  float acc[8][8], slab[8][8], total[8][8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[i][j] = slab[i][j] = total[i][j] = 0.f;

  // a thread stages rows tid / 4 and 64 + tid / 4 of both operands, k (tid % 4) * 4 .. + 3 of the tile
  const int lr = tid / 4, lk = (tid % 4) * 4;
  float ra[2][4], rw[2][4];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      fetch4<TA>(A, lda, m0 + h * 64 + lr, M, k0 + lk, K, a_vector_ok, ra[h]);
      fetch4<TW>(W, K, n0 + h * 64 + lr, N, k0 + lk, K, w_vector_ok, rw[h]);
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        As[buf][lk + e][h * 64 + lr] = ra[h][e];
        Ws[buf][lk + e][h * 64 + lr] = rw[h][e];
      }
  };
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += BK) {
    const bool more = k0 + BK < K;
    if (more) fetch(k0 + BK);
#pragma unroll 4
    for (int kk = 0; kk < BK; ++kk) {
      float a[8], w[8];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const f32x4_t av = *(const f32x4_t*)&As[buf][kk][h * 64 + ty * 4];
        const f32x4_t wv = *(const f32x4_t*)&Ws[buf][kk][h * 64 + tx * 4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[h * 4 + e] = av[e];
          w[h * 4 + e] = wv[e];
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    if (more) stage(buf ^ 1);
    __syncthreads();
    buf ^= 1;
    const int done = k0 + BK;
    if (done % RANGE_K == 0 || done >= K) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          slab[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    if (done % SLAB_K == 0 || done >= K) {
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          total[i][j] += slab[i][j];
          slab[i][j] = 0.f;
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int m = m0 + (i / 4) * 64 + ty * 4 + i % 4;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int n = n0 + (j / 4) * 64 + tx * 4 + j % 4;
      if (n >= N) continue;
      float v = total[i][j];
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
  // the wide tiles where they are enough to occupy a quarter of the GPU at least (2,048 x 37,888 x 3,584: 7.9 ms
  // against 15.1, 90 % of the rate of unpacked FMAs; 200 x 1,000 x 520, 16 tiles: 107 us against 81)
  const long long wide_tiles = (long long)((M + WIDE - 1) / WIDE) * ((N + WIDE - 1) / WIDE);
  if (M >= WIDE && N >= WIDE && wide_tiles >= 64) {
    dim3 grid((N + WIDE - 1) / WIDE, (M + WIDE - 1) / WIDE);
    // 16-byte loads where every row of an operand starts on a 16-byte boundary
    const int a_ok = sizeof(TA) == 4 && ((uintptr_t)A % 16 == 0) && lda % 4 == 0;
    const int w_ok = sizeof(TW) == 4 && ((uintptr_t)W % 16 == 0) && K % 4 == 0;
    if (accumulate)
      gemm_generic_wide_kernel<TA, TW, TC, true><<<grid, 256, 0, s>>>((const TA*)A, (const TW*)W, bias, (TC*)C, M, N, K, lda,
                                                                      ldc, a_ok, w_ok);
    else
      gemm_generic_wide_kernel<TA, TW, TC, false><<<grid, 256, 0, s>>>((const TA*)A, (const TW*)W, bias, (TC*)C, M, N, K, lda,
                                                                       ldc, a_ok, w_ok);
    VK_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (accumulate)
    gemm_generic_kernel<TA, TW, TC, true><<<grid, 256, 0, s>>>((const TA*)A, (const TW*)W, bias, (TC*)C, M, N, K, lda, ldc);
  else
    gemm_generic_kernel<TA, TW, TC, false><<<grid, 256, 0, s>>>((const TA*)A, (const TW*)W, bias, (TC*)C, M, N, K, lda, ldc);
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// The weight stream, for 32-bit A and W and up to 64 rows of A. A workgroup of four waves owns 64 rows
// of W and one slab of K; wave w owns range w of the slab, and each of its lanes one row of W, whose
// chain over the range's k it computes for all rows of A (MT accumulators). What a lane needs of W is
// consecutive in memory, which is the opposite of what 64 lanes should request together: so W goes
// through LDS, in stages of 32 k (8 KB per wave): a wave's load instruction fetches eight rows' 128 bytes
// each and writes them straight into LDS (no registers in between), the next stage's instructions in
// flight while this stage is multiplied. Rows are 128 bytes in LDS and cannot be padded (a load writes
// lane L's 16 bytes at 16 L), so chunk c of row r sits in slot c ^ (r / 2 % 8): the 16 lanes that read
// together then touch 16 different 16-byte bank groups. The stage's columns of A come the same way and
// are read by all lanes at one address (a broadcast). A wave has one stage of loads in flight while it
// multiplies the other, and the waves do not wait for one another until the end of the range.
constexpr int STREAM_ROWS = 64, SUB_K = 32, W_STAGE = STREAM_ROWS * SUB_K * 4, W_LOADS = W_STAGE / 1024;

typedef __attribute__((address_space(3))) void* lds_ptr;
typedef __attribute__((address_space(1))) const void* global_ptr;

// Until at most N of the wave's vector memory loads are in flight (they complete in the order of their issue).
// Also a barrier for the compiler: no LDS read may move above the wait for the load that fills what it reads,
// and none below the issue of the load that overwrites it.
template <int N>
__device__ __forceinline__ void wait_loads_but() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int MT>
__global__ __launch_bounds__(256) void gemm_stream_kernel(const float* __restrict__ A, const float* __restrict__ W,
                                                          float* __restrict__ slabs, int M, int N, int K,
                                                          long long lda) {
  constexpr int A_LOADS = (MT + 7) / 8;                 // a load instruction brings 32 k of eight rows of A
  constexpr int STAGE = W_STAGE + A_LOADS * 1024;
  constexpr int LOADS = W_LOADS + A_LOADS;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int n0 = blockIdx.x * STREAM_ROWS, slab = blockIdx.y;
  const int k_begin = slab * SLAB_K + wave * RANGE_K;
  const int k_end = min(K, k_begin + RANGE_K);           // K is a multiple of 4
  unsigned char* mine = lds + wave * 2 * STAGE;
  float acc[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc[m] = 0.f;

  // what this lane fetches with each load instruction of a stage: of W, chunk (slot ^ swizzle) of row 8 i + sub_row;
  // of A, chunk `slot` of row 8 i + sub_row. A row past the end is a copy of the last one and is not stored; a
  // chunk past the end of K is a copy of the last one and is never multiplied.
  const int sub_row = lane >> 3, slot = lane & 7;
  const float* w_from[W_LOADS];
  int w_chunk[W_LOADS];
#pragma unroll
  for (int i = 0; i < W_LOADS; ++i) {
    const int r = i * 8 + sub_row;
    w_from[i] = W + (size_t)min(n0 + r, N - 1) * K;
    w_chunk[i] = (slot ^ ((r >> 1) & 7)) << 2;
  }
  auto issue = [&](int k_sub, int stage) {
    unsigned char* to = mine + stage * STAGE;
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i)
      __builtin_amdgcn_global_load_lds((global_ptr)(w_from[i] + min(k_sub + w_chunk[i], K - 4)),
                                       (lds_ptr)(to + i * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_ptr)(A + (size_t)min(i * 8 + sub_row, M - 1) * lda + min(k_sub + (slot << 2), K - 4)),
          (lds_ptr)(to + W_STAGE + i * 1024), 16, 0, 0);
  };
  const unsigned my_row = (unsigned)(lane * (SUB_K * 4)), my_swizzle = (unsigned)((lane >> 1) & 7);
  if (k_begin < k_end) {
    const int subs = (k_end - k_begin + SUB_K - 1) / SUB_K;
    issue(k_begin, 0);
    for (int s = 0; s < subs; ++s) {
      const int k_sub = k_begin + s * SUB_K;
      if (s + 1 < subs) {
        issue(k_sub + SUB_K, (s + 1) & 1);   // that stage was multiplied in the step before this one
        wait_loads_but<LOADS>();
      } else {
        wait_loads_but<0>();
      }
      const unsigned char* stage = mine + (s & 1) * STAGE;
      const int chunks = (min(k_end, k_sub + SUB_K) - k_sub) >> 2;
      if (chunks == SUB_K / 4) {
#pragma unroll
        for (int j = 0; j < SUB_K / 4; ++j) {
          const f32x4_t w = *(const f32x4_t*)(stage + my_row + ((j ^ my_swizzle) << 4));
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const f32x4_t a = *(const f32x4_t*)(stage + W_STAGE + m * (SUB_K * 4) + (j << 4));   // the same for every lane
            acc[m] = fmaf(a[0], w[0], acc[m]);
            acc[m] = fmaf(a[1], w[1], acc[m]);
            acc[m] = fmaf(a[2], w[2], acc[m]);
            acc[m] = fmaf(a[3], w[3], acc[m]);
          }
        }
      } else {
        for (int j = 0; j < chunks; ++j) {
          const f32x4_t w = *(const f32x4_t*)(stage + my_row + ((j ^ my_swizzle) << 4));
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            const f32x4_t a = *(const f32x4_t*)(stage + W_STAGE + m * (SUB_K * 4) + (j << 4));
            acc[m] = fmaf(a[0], w[0], acc[m]);
            acc[m] = fmaf(a[1], w[1], acc[m]);
            acc[m] = fmaf(a[2], w[2], acc[m]);
            acc[m] = fmaf(a[3], w[3], acc[m]);
          }
        }
      }
      // the next step's loads overwrite the other stage, which the step before this one read: its reads are done,
      // since their values went into the chains above; nothing of this step may move below the next issue
      asm volatile("" ::: "memory");
    }
  }
  // the slab's sum: the four ranges in ascending order, through LDS (every wave is done with its stages)
  __syncthreads();
  float* sums = (float*)lds;   // [wave][m][row]
#pragma unroll
  for (int m = 0; m < MT; ++m) sums[(wave * MT + m) * STREAM_ROWS + lane] = acc[m];
  __syncthreads();
  for (int at = threadIdx.x; at < MT * STREAM_ROWS; at += 256) {
    const int m = at / STREAM_ROWS, r = at % STREAM_ROWS;
    if (m >= M || n0 + r >= N) continue;
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < SLAB_RANGES; ++w) total += sums[(w * MT + m) * STREAM_ROWS + r];
    slabs[((size_t)slab * M + m) * N + n0 + r] = total;
  }
}

// C = +0 + slab 0 + slab 1 + ... (+ bias) (+ old C): the last level of the sum.
template <typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_stream_finish_kernel(const float* __restrict__ slabs,
                                                                 const float* __restrict__ bias, TC* __restrict__ C,
                                                                 int M, int N, long long ldc, int num_slabs) {
  const long long at = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (at >= (long long)M * N) return;
  const int m = (int)(at / N), n = (int)(at % N);
  float total = 0.f;
  for (int s = 0; s < num_slabs; ++s) total += slabs[(size_t)s * M * N + at];
  if (bias) total += bias[n];
  TC* dst = C + (size_t)m * ldc + n;
  if (ACCUMULATE)
    *dst = from_float<TC>(to_float<TC>(*dst) + total);
  else
    *dst = from_float<TC>(total);
}

template <int MT>
int launch_stream_as(const float* A, const float* W, float* slabs, int M, int N, int K, long long lda, int num_slabs,
                     hipStream_t s) {
  constexpr int lds_bytes = 4 * 2 * (W_STAGE + (MT + 7) / 8 * 1024);
  static_assert(4 * MT * STREAM_ROWS * 4 <= lds_bytes, "the ranges' sums reuse the stages");
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_stream_kernel<MT>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                       lds_bytes);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  dim3 grid((N + STREAM_ROWS - 1) / STREAM_ROWS, num_slabs);
  gemm_stream_kernel<MT><<<grid, 256, lds_bytes, s>>>(A, W, slabs, M, N, K, lda);
  VK_LAUNCH_CHECK();
  return 0;
}
}  // namespace

// Floats of workspace that vk_gemm_stream needs for an M x N product over K.
extern "C" long long vk_gemm_stream_workspace(int M, int N, int K) {
  return (long long)((K + SLAB_K - 1) / SLAB_K) * M * N;
}

// The weight stream: float A (row stride lda, a multiple of 4) and W, M <= 64, K a multiple of 4, 16-byte aligned
// operands; C float or bfloat16. `slabs`: workspace of vk_gemm_stream_workspace(M, N, K) floats.
extern "C" int vk_gemm_stream(const float* A, const float* W, const float* bias, void* C, int c_dtype, int M, int N,
                              int K, long long lda, long long ldc, int accumulate, float* slabs,
                              long long slab_floats, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 64) return VK_UNSUPPORTED_SIZE;
  if (K < 4 || (K & 3) || (lda & 3) || lda < K || ldc < N || !slabs) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (accumulate && c_dtype != DT_F32) return VK_BAD_ARGUMENT;
  const int num_slabs = (K + SLAB_K - 1) / SLAB_K;
  if ((long long)num_slabs * M * N > slab_floats || num_slabs > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  int status;
  if (M <= 1) status = launch_stream_as<1>(A, W, slabs, M, N, K, lda, num_slabs, s);
  else if (M <= 2) status = launch_stream_as<2>(A, W, slabs, M, N, K, lda, num_slabs, s);
  else if (M <= 4) status = launch_stream_as<4>(A, W, slabs, M, N, K, lda, num_slabs, s);
  else if (M <= 8) status = launch_stream_as<8>(A, W, slabs, M, N, K, lda, num_slabs, s);
  else if (M <= 16) status = launch_stream_as<16>(A, W, slabs, M, N, K, lda, num_slabs, s);
  else if (M <= 32) status = launch_stream_as<32>(A, W, slabs, M, N, K, lda, num_slabs, s);
  else status = launch_stream_as<64>(A, W, slabs, M, N, K, lda, num_slabs, s);
  if (status != 0) return status;
  const long long outputs = (long long)M * N;
  const unsigned blocks = (unsigned)((outputs + 255) / 256);
  if (c_dtype == DT_F32) {
    if (accumulate)
      gemm_stream_finish_kernel<float, true><<<blocks, 256, 0, s>>>(slabs, bias, (float*)C, M, N, ldc, num_slabs);
    else
      gemm_stream_finish_kernel<float, false><<<blocks, 256, 0, s>>>(slabs, bias, (float*)C, M, N, ldc, num_slabs);
  } else if (c_dtype == DT_BF16) {
    gemm_stream_finish_kernel<bf16_t, false><<<blocks, 256, 0, s>>>(slabs, bias, (bf16_t*)C, M, N, ldc, num_slabs);
  } else {
    return VK_BAD_ARGUMENT;
  }
  VK_LAUNCH_CHECK();
  return 0;
}

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
