// bfloat16 matrix products on the matrix cores of gfx950: C[M,N] (+)= A[M,K] * W[N,K]^T (+ bias[N]),
// products in bfloat16, sums in 32-bit (v_mfma_f32_16x16x32_bf16).
//
// Both operands are contiguous along K, which is how that instruction wants them: a lane holds 8
// consecutive k of one row. The weight tile is the instruction's first operand and the activation
// tile the second, so a lane ends up with four consecutive output columns of one token and can store
// them as one vector:
//     lane l, register j of an accumulator  <->  C[token l % 16][column 4 * (l / 16) + j]
//
// Two kernels:
//   gemm_tile    M large (prompts). 128x128 output tile per workgroup of four waves, K in steps of 64
//                staged through LDS (rows padded to 144 bytes, which spreads the 16-byte reads of 16
//                rows over all banks), double-buffered, one barrier per step. Workgroups are renumbered
//                so that those running on one XCD (one L2) work on neighbouring tiles.
//   gemm_skinny  M <= 64 (decoding). The product is a stream of the weights from HBM: a workgroup owns
//                16 weight rows, its four waves split K in interleaved spans of 128 and read their span
//                straight into the instruction's operand layout (no LDS), two spans in flight; the four
//                partial sums are added in a fixed order.
// Every sum has one fixed order for a given shape.
//
// Reference for what is computed: crates/vipera-backend-cpu/src/model.rs:1005-1031 (batched products,
// bias after the product); the idea of reading a weight row once for many tokens is that of the
// reference's batched matvec (crates/vipera-backend-gpu/src/q4k_matvec_q8_batch.cu:40-116).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

template <typename TC, bool ACCUMULATE>
__device__ __forceinline__ void store4(TC* __restrict__ C, long long ldc, int m, int n, int M, int N, f32x4 v,
                                       const float* __restrict__ bias, bool vector_ok) {
  if (m >= M || n >= N) return;
  TC* dst = C + (size_t)m * ldc + n;
  if (vector_ok && n + 3 < N) {
    if (bias) {
      const f32x4 b = *(const f32x4*)(bias + n);
      v += b;
    }
    if constexpr (sizeof(TC) == 4) {
      f32x4* p = (f32x4*)dst;
      if (ACCUMULATE) v += *p;
      *p = v;
    } else {
      bf16x4 o;
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = (__bf16)v[j];
      *(bf16x4*)dst = o;
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    if (n + j >= N) break;
    float x = v[j];
    if (bias) x += bias[n + j];
    if (ACCUMULATE) x += to_float<TC>(dst[j]);
    dst[j] = from_float<TC>(x);
  }
}

// ---------------------------------------------------------------------------------------------
constexpr int BM = 128, BN = 128, BK = 64;
constexpr int ROW = BK + 8;  // elements per LDS row: 144 bytes
constexpr int TILE_ELEMS = BM * ROW;
constexpr int XCDS = 8;

template <typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(256) void gemm_tile_kernel(const __bf16* __restrict__ A, const __bf16* __restrict__ W,
                                                        const float* __restrict__ bias, TC* __restrict__ C, int M,
                                                        int N, int K, long long lda, long long ldc, int tiles_m,
                                                        int tiles_n, int vector_ok) {
  extern __shared__ __attribute__((aligned(16))) __bf16 lds[];
  __bf16* sA = lds;                   // [2][BM][ROW]
  __bf16* sW = lds + 2 * TILE_ELEMS;  // [2][BN][ROW]

  // workgroups are dealt to the XCDs round-robin; give each XCD a contiguous run of tiles
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + XCDS - 1) / XCDS;
  const int logical = (blockIdx.x % XCDS) * per_xcd + blockIdx.x / XCDS;
  if (logical >= total) return;
  // tiles of one column panel of W (all m for one n) are neighbours
  const int tile_n = logical / tiles_m, tile_m = logical % tiles_m;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int lr = lane & 15, lg = lane >> 4;

  f32x4 acc[4][4];  // [n tile][m tile]
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // staging: 1024 chunks of 16 bytes per operand tile, four per thread
  bf16x8 ra[4], rw[4];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = tid + 256 * i;
      const int row = id >> 3, c = id & 7;
      const int k = k0 + c * 8;
      const int am = m0 + row, wn_ = n0 + row;
      ra[i] = (am < M && k < K) ? *(const bf16x8*)(A + (size_t)am * lda + k) : zero8();
      rw[i] = (wn_ < N && k < K) ? *(const bf16x8*)(W + (size_t)wn_ * K + k) : zero8();
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int id = tid + 256 * i;
      const int row = id >> 3, c = id & 7;
      *(bf16x8*)(sA + buf * TILE_ELEMS + row * ROW + c * 8) = ra[i];
      *(bf16x8*)(sW + buf * TILE_ELEMS + row * ROW + c * 8) = rw[i];
    }
  };

  const int steps = (K + BK - 1) / BK;
  load_global(0);
  store_lds(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) load_global((s + 1) * BK);
    const __bf16* tA = sA + buf * TILE_ELEMS + (wm * 64 + lr) * ROW + lg * 8;
    const __bf16* tW = sW + buf * TILE_ELEMS + (wn * 64 + lr) * ROW + lg * 8;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      bf16x8 fa[4], fw[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        fa[t] = *(const bf16x8*)(tA + t * 16 * ROW + ks * 32);
        fw[t] = *(const bf16x8*)(tW + t * 16 * ROW + ks * 32);
      }
#pragma unroll
      for (int tn = 0; tn < 4; ++tn)
#pragma unroll
        for (int tm = 0; tm < 4; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[tn], fa[tm], acc[tn][tm], 0, 0, 0);
    }
    if (s + 1 < steps) store_lds(buf ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int tn = 0; tn < 4; ++tn)
#pragma unroll
    for (int tm = 0; tm < 4; ++tm)
      store4<TC, ACCUMULATE>(C, ldc, m0 + wm * 64 + tm * 16 + lr, n0 + wn * 64 + tn * 16 + lg * 4, M, N, acc[tn][tm],
                             bias, vector_ok != 0);
}

// ---------------------------------------------------------------------------------------------
constexpr int SPAN = 128;  // k per wave per step: four instructions of 32

// CB: blocks of 16 tokens (M <= 16 * CB). RT: tiles of 16 weight rows per wave. WAVES: waves of a
// workgroup, which split K in interleaved spans. A workgroup owns 16 * RT weight rows.
template <int CB, int RT, int WAVES, typename TC, bool ACCUMULATE>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const __bf16* __restrict__ A,
                                                                  const __bf16* __restrict__ W,
                                                                  const float* __restrict__ bias,
                                                                  TC* __restrict__ C, int M, int N, int K,
                                                                  long long lda, long long ldc, int vector_ok) {
  __shared__ f32x4 partial[WAVES][RT * CB][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int lr = lane & 15, lg = lane >> 4;
  const int n0 = blockIdx.x * 16 * RT;
  const __bf16* wp[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int wrow = min(n0 + rt * 16 + lr, N - 1);  // rows past N are read from the last row and never stored
    wp[rt] = W + (size_t)wrow * K + lg * 8;
  }
  const __bf16* ap[CB];
  bool a_ok[CB];
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) {
    const int m = cb * 16 + lr;
    a_ok[cb] = m < M;
    ap[cb] = A + (size_t)(a_ok[cb] ? m : 0) * lda + lg * 8;
  }
  f32x4 acc[RT][CB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) acc[rt][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int spans = (K + SPAN - 1) / SPAN;
  // two spans are in flight: while one is multiplied, the loads of the next (weights and activations)
  // are already issued, and nothing of the current span waits for them
  bf16x8 w_cur[RT][4], w_next[RT][4], a_cur[CB][4], a_next[CB][4];
  auto load_span = [&](int span, bf16x8 (*w_dst)[4], bf16x8 (*a_dst)[4]) {
    const int kb = span * SPAN;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const bool ok = span < spans && kb + i * 32 + lg * 8 < K;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) w_dst[rt][i] = ok ? *(const bf16x8*)(wp[rt] + kb + i * 32) : zero8();
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) a_dst[cb][i] = (ok && a_ok[cb]) ? *(const bf16x8*)(ap[cb] + kb + i * 32) : zero8();
    }
  };
  load_span(wave, w_cur, a_cur);
  for (int span = wave; span < spans; span += WAVES) {
    load_span(span + WAVES, w_next, a_next);
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_cur[rt][i], a_cur[cb][i], acc[rt][cb], 0, 0, 0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) w_cur[rt][i] = w_next[rt][i];
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) a_cur[cb][i] = a_next[cb][i];
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) partial[wave][rt * CB + cb][lane] = acc[rt][cb];
  __syncthreads();
  // the waves share out the tiles; every tile's partial sums are added in wave order
  for (int t = wave; t < RT * CB; t += WAVES) {
    f32x4 sum = partial[0][t][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) sum += partial[w][t][lane];
    const int rt = t / CB, cb = t % CB;
    store4<TC, ACCUMULATE>(C, ldc, cb * 16 + lr, n0 + rt * 16 + lg * 4, M, N, sum, bias, vector_ok != 0);
  }
}

template <int CB, int RT, int WAVES, typename TC, bool ACC>
int launch_skinny_as(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                     long long ldc, int vector_ok, hipStream_t s) {
  const int blocks = (N + 16 * RT - 1) / (16 * RT);
  gemm_skinny_kernel<CB, RT, WAVES, TC, ACC><<<blocks, WAVES * 64, 0, s>>>(A, W, bias, C, M, N, K, lda, ldc, vector_ok);
  VK_LAUNCH_CHECK();
  return 0;
}

// Shape of the launch: few weight rows (N / 16 tiles below `many`) want many waves per workgroup so
// that enough loads are in flight; many rows want more rows per wave so that activations are re-read less.
template <int CB, typename TC, bool ACC>
int launch_skinny_cb(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                     long long ldc, int vector_ok, int shape, hipStream_t s) {
  const int tiles = (N + 15) / 16;
  // measured on the 7B shapes; sixteen waves with more than one token block would not fit the registers
  if (shape == 0) shape = tiles >= 1024 ? ((CB >= 2 || M > 4) ? 2 : 1) : (CB == 1 ? 3 : 1);
  switch (shape) {
    case 1: return launch_skinny_as<CB, 1, 4, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, s);
    case 2: return launch_skinny_as<CB, 2, 4, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, s);
    case 3: return launch_skinny_as<CB, 1, 16, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, s);
    case 4: return launch_skinny_as<CB, 1, 8, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, s);
    case 5: return launch_skinny_as<CB, 2, 8, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, s);
  }
  return VK_BAD_ARGUMENT;
}

template <typename TC, bool ACC>
int launch_skinny(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                  long long ldc, int vector_ok, int shape, hipStream_t s) {
  switch ((M + 15) / 16) {
    case 1: return launch_skinny_cb<1, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, shape, s);
    case 2: return launch_skinny_cb<2, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, shape, s);
    case 3: return launch_skinny_cb<3, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, shape, s);
    case 4: return launch_skinny_cb<4, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, shape, s);
  }
  return VK_UNSUPPORTED_SIZE;
}

template <typename TC, bool ACC>
int launch_tile(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                long long ldc, int vector_ok, hipStream_t s) {
  static bool configured = false;
  constexpr int lds_bytes = 4 * TILE_ELEMS * (int)sizeof(__bf16);
  auto kernel = gemm_tile_kernel<TC, ACC>;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const long long total = (long long)tiles_m * tiles_n;
  const long long grid = (total + XCDS - 1) / XCDS * XCDS;
  if (grid > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  kernel<<<(int)grid, 256, lds_bytes, s>>>(A, W, bias, C, M, N, K, lda, ldc, tiles_m, tiles_n, vector_ok);
  VK_LAUNCH_CHECK();
  return 0;
}
}  // namespace

// A, W: bfloat16. c_dtype: 0 float, 1 bfloat16. accumulate needs a float C. Requirements (checked here):
// K a multiple of 8 and lda a multiple of 8 (16-byte chunks); A and W 16-byte aligned.
// `skinny_limit`: M at or below it takes the weight-streaming kernel (at most 64).
// `skinny_shape`: 0 lets the launcher choose rows per wave and waves per workgroup; 1..5 force a choice.
extern "C" int vk_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N, int K,
                            long long lda, long long ldc, int accumulate, int skinny_limit, int skinny_shape, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (accumulate && c_dtype != DT_F32) return VK_BAD_ARGUMENT;
  const int elem = c_dtype == DT_F32 ? 4 : 2;
  const int vector_ok = ((ldc & 3) == 0 && ((uintptr_t)C & (4 * elem - 1)) == 0 &&
                         (bias == nullptr || ((uintptr_t)bias & 15) == 0)) ? 1 : 0;
  hipStream_t s = (hipStream_t)stream;
  const __bf16* a = (const __bf16*)A;
  const __bf16* w = (const __bf16*)W;
  const bool skinny = M <= (skinny_limit < 64 ? skinny_limit : 64);
  if (c_dtype == DT_F32) {
    if (accumulate)
      return skinny ? launch_skinny<float, true>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, skinny_shape, s)
                    : launch_tile<float, true>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, s);
    return skinny ? launch_skinny<float, false>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, skinny_shape, s)
                  : launch_tile<float, false>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, s);
  }
  if (c_dtype == DT_BF16)
    return skinny ? launch_skinny<__bf16, false>(a, w, bias, (__bf16*)C, M, N, K, lda, ldc, vector_ok, skinny_shape, s)
                  : launch_tile<__bf16, false>(a, w, bias, (__bf16*)C, M, N, K, lda, ldc, vector_ok, s);
  return VK_BAD_ARGUMENT;
}
