// bfloat16 matrix products on the matrix cores of gfx950: C[M,N] (+)= A[M,K] * W[N,K]^T (+ bias[N]),
// products in bfloat16, sums in 32-bit (v_mfma_f32_16x16x32_bf16).
//
// Both operands are contiguous along K, which is how that instruction wants them: a lane holds 8
// consecutive k of one row. The weight tile is the instruction's first operand and the activation
// tile the second, so a lane ends up with four consecutive output columns of one token and can store
// them as one vector:
//     lane l, register j of an accumulator  <->  C[token l % 16][column 4 * (l / 16) + j]
//
// Kernels:
//   gemm_tile    more than 64 tokens (prompts). An output tile per workgroup (256x256 down to 128x128,
//                chosen with a split of K by an estimate of the time), K in steps of 64 through two LDS
//                stages, one barrier per step. Workgroups are renumbered so that those running on one XCD
//                (one L2) work on neighbouring tiles. Two kernels: gemm_tile_direct_kernel loads both
//                operands straight into LDS (unpadded rows, chunks swizzled) and pipelines the LDS reads
//                against the products inside each wave; it takes K in multiples of 64. gemm_tile_kernel
//                stages the operands through registers into rows padded to 144 bytes and takes any K that
//                is a multiple of 8.
//   gemm_skinny  a few tokens (decoding). The product is a stream of the weights from HBM: a workgroup
//                owns 16 weight rows, its waves split K in interleaved spans of 128 and read their span
//                straight into the instruction's operand layout (no LDS); the waves' partial sums are
//                added in a fixed order.
//   gemm_mid     up to 64 tokens. The same stream of weights, with the activations of a 256-wide chunk
//                of K fetched once per workgroup into LDS; K may be split over workgroups, whose partial
//                sums a second kernel adds in a fixed order.
// The two streaming kernels read through buffer descriptors, so that no load sits behind a branch, and
// rotate their operand register sets at compile time (pipeline.h): a use waits for exactly its own
// loads and the loads of the next spans stay in flight. The gated epilogue of gemm_tile and gemm_mid
// turns the fused gate/up product into up * silu(gate).
// Every sum has one fixed order for a given shape.
//
// Reference for what is computed: crates/vipera-backend-cpu/src/model.rs:1005-1031 (batched products,
// bias after the product); the idea of reading a weight row once for many tokens is that of the
// reference's batched matvec (crates/vipera-backend-gpu/src/q4k_matvec_q8_batch.cu:40-116).
#include <cmath>
#include <mutex>

#include "common.h"
#include "no_alloc.h"
#include "pipeline.h"

// Depth of the load pipelines of the weight-streaming kernels: register sets of operands, one being
// multiplied while the others are in flight (measured on an MI355X).
#ifndef VK_SKINNY_SETS
#define VK_SKINNY_SETS 3
#endif
#ifndef VK_MID_SETS
#define VK_MID_SETS 3
#endif

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

// A range of memory behind a buffer descriptor (wave-uniform): a 16-byte read at a byte offset at or
// past `bytes` returns zero without touching memory. Offsets and sizes are 32-bit.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
struct BufferView {
  __amdgpu_buffer_rsrc_t rsrc;
  __device__ __forceinline__ bf16x8 load(unsigned byte_offset) const {
    return __builtin_bit_cast(bf16x8, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)byte_offset, 0, 0));
  }
};
__device__ __forceinline__ BufferView buffer_view(const void* base, unsigned long long bytes) {
  const unsigned range = bytes > 0xffffffffull ? 0xffffffffu : (unsigned)bytes;
  // third word: raw buffer, 32-bit data format (what the compiler's own buffer accesses use on gfx9)
  return BufferView{__builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)range, 0x00020000)};
}

typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

// Four consecutive outputs of row m from column n on, columns at or past N left out. `align`: 4 when the
// four may go as one vector (C, its row stride and the bias aligned to four elements and n a multiple of
// four), 2 when pairs may (n even), else element by element.
template <typename TC, bool ACCUMULATE>
__device__ __forceinline__ void store4_aligned(TC* __restrict__ C, long long ldc, int m, int n, int M, int N, f32x4 v,
                                               const float* __restrict__ bias, int align);

template <typename TC, bool ACCUMULATE>
__device__ __forceinline__ void store4(TC* __restrict__ C, long long ldc, int m, int n, int M, int N, f32x4 v,
                                       const float* __restrict__ bias, bool vector_ok) {
  store4_aligned<TC, ACCUMULATE>(C, ldc, m, n, M, N, v, bias, vector_ok ? 4 : 1);
}

template <typename TC, bool ACCUMULATE>
__device__ __forceinline__ void store4_aligned(TC* __restrict__ C, long long ldc, int m, int n, int M, int N, f32x4 v,
                                               const float* __restrict__ bias, int align) {
  if (m >= M || n >= N) return;
  TC* dst = C + (size_t)m * ldc + n;
  if (align == 2) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int nn = n + 2 * h;
      if (nn + 1 < N) {
        f32x2 x = {v[2 * h], v[2 * h + 1]};
        if (bias) x += *(const f32x2*)(bias + nn);
        if constexpr (sizeof(TC) == 4) {
          f32x2* p = (f32x2*)(dst + 2 * h);
          if (ACCUMULATE) x += *p;
          *p = x;
        } else {
          bf16x2 o = {(__bf16)x[0], (__bf16)x[1]};
          *(bf16x2*)(dst + 2 * h) = o;
        }
      } else if (nn < N) {
        float x = v[2 * h];
        if (bias) x += bias[nn];
        if (ACCUMULATE) x += to_float<TC>(dst[2 * h]);
        dst[2 * h] = from_float<TC>(x);
      }
    }
    return;
  }
  const bool vector_ok = align == 4;
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

// The gated epilogue. The fused gate/up weight interleaves its rows in groups of 16: fused rows
// [32 p, 32 p + 16) are gate rows [16 p, 16 p + 16) and fused rows [32 p + 16, 32 p + 32) are the up rows of
// the same outputs. A pair of accumulators (gate, up) of one token block gives
// out[m][16 p + 4 g + j] = up * gate / (1 + exp(-gate)) (crates/vipera-backend-cpu/src/model.rs:4368-4374).
__device__ __forceinline__ void store_gated(__bf16* __restrict__ C, long long ldc, int m, int n, int M, int inter,
                                            f32x4 gate, f32x4 up) {
  if (m >= M || n >= inter) return;
  __bf16* dst = C + (size_t)m * ldc + n;
  bf16x4 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = (__bf16)(up[j] * (gate[j] / (1.0f + __expf(-gate[j]))));
  if (n + 3 < inter && (ldc & 3) == 0 && ((uintptr_t)C & 7) == 0) {
    *(bf16x4*)dst = o;
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (n + j < inter) dst[j] = o[j];
  }
}

// ---------------------------------------------------------------------------------------------
constexpr int BK = 64;
constexpr int ROW = BK + 8;  // elements per LDS row: 144 bytes
constexpr int XCDS = 8;

// The second half of an RMS norm that is split between the products around it (see FollowNorm), in a tiled
// product, for any number of tokens: the input is x * gain as the product before the norm left it, and the 32-bit
// sums of token m are multiplied by 1 / sqrt(sum over the groups of sumsq[group * stride + m] / K + eps) before
// bias and activation. The first half stays with the kernels of up to 64 tokens: in the tiled kernel's epilogue it
// was measured too (x * gain and the squares of each wave's columns written beside the residual) and saves
// nothing from 128 to 2,048 tokens, where the norm kernel it replaces moves little more than the epilogue adds.
struct TileNorm {
  const float* sumsq = nullptr;
  int groups = 0, stride = 0;
  float eps = 0.f;
};

// At the start of a tile kernel the THREADS / BM threads of a token each add every
// (THREADS / BM)-th group, in ascending order, and leave their part in part_sums[part * BM + token] (a token past M
// takes the last one's, which nothing uses). A thread requests 32 groups at a time at clamped addresses before it
// adds any: one round trip to memory for up to 64 groups on two threads, behind the tile's first operand requests,
// where a loop of a load and an addition at a time cost the gate/up product of 2,048 tokens 69 us of 437. The
// barrier before the first product makes the parts visible; tile_norm_factor adds them in ascending order.
template <int BM, int THREADS>
__device__ __forceinline__ void tile_norm_parts(const TileNorm& norm, int m0, int M, int tid, float* part_sums) {
  static_assert(THREADS % BM == 0, "whole threads per token");
  constexpr int PER = THREADS / BM, AHEAD = 32;
  if (!norm.sumsq) return;
  const int token = tid % BM, part = tid / BM;
  const float* of_token = norm.sumsq + min(m0 + token, M - 1);
  float squares = 0.f;
  for (int base = part; base < norm.groups; base += AHEAD * PER) {
    float ahead[AHEAD];
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) ahead[j] = of_token[(size_t)min(base + j * PER, norm.groups - 1) * norm.stride];
#pragma unroll
    for (int j = 0; j < AHEAD; ++j)
      if (base + j * PER < norm.groups) squares += ahead[j];
  }
  part_sums[part * BM + token] = squares;
}
template <int BM, int THREADS>
__device__ __forceinline__ float tile_norm_factor(const TileNorm& norm, const float* part_sums, int token, int K) {
  float squares = 0.f;
#pragma unroll
  for (int part = 0; part < THREADS / BM; ++part) squares += part_sums[part * BM + token];
  return 1.0f / sqrtf(squares / (float)K + norm.eps);
}

// What a wave of a tile kernel does with its sums: acc[tn][tm] holds, in lane (lr, lg), outputs
// [wave_n + tn * 16 + lg * 4, + 4) of token wave_m + tm * 16 + lr. `part_sums`: see tile_norm_parts; `wave_token`:
// the wave's first token within the tile.
template <int BM, int THREADS, int TM, int TN, typename TC, bool ACCUMULATE, bool GATED>
__device__ __forceinline__ void tile_epilogue(f32x4 (&acc)[TN][TM], TC* __restrict__ C, long long ldc, int M, int N,
                                              int K, const float* __restrict__ bias, bool vector_ok, int wave_m,
                                              int wave_n, int lr, int lg, const TileNorm& norm,
                                              const float* part_sums, int wave_token) {
  if (norm.sumsq) {
#pragma unroll
    for (int tm = 0; tm < TM; ++tm) {
      const float inv = tile_norm_factor<BM, THREADS>(norm, part_sums, wave_token + tm * 16 + lr, K);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn) acc[tn][tm] *= inv;
    }
  }
  if constexpr (GATED) {
    // N counts fused rows (pairs of 16-row tiles: gate, up); the output has N / 2 columns
    static_assert(!GATED || TN % 2 == 0, "a wave must own whole gate/up pairs");
#pragma unroll
    for (int pair = 0; pair < TN / 2; ++pair)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        store_gated((__bf16*)C, ldc, wave_m + tm * 16 + lr, (wave_n + pair * 32) / 2 + lg * 4, M, N / 2,
                    acc[2 * pair][tm], acc[2 * pair + 1][tm]);
    return;
  }
#pragma unroll
  for (int tn = 0; tn < TN; ++tn)
#pragma unroll
    for (int tm = 0; tm < TM; ++tm)
      store4<TC, ACCUMULATE>(C, ldc, wave_m + tm * 16 + lr, wave_n + tn * 16 + lg * 4, M, N, acc[tn][tm], bias, vector_ok);
}

// Which tile the `logical`-th workgroup of a launch owns. An XCD gets a contiguous run of logical numbers, and the
// tiles of a run share that XCD's L2: the numbers walk blocks of `group_m` tile rows, down the rows of a block first
// and then along its columns, so that a run covers few rows of tiles of A and few of W at the same time (a run of
// 28 tiles of 256 x 128 as 4 x 7 reads 1,024 rows of A and 896 of W at every step of K, as 8 x 3.5 2,048 and 448:
// a quarter fewer bytes into L2). The last block may have fewer rows.
__device__ __forceinline__ void tile_of(int logical, int tiles_m, int tiles_n, int group_m, int* tile_m, int* tile_n) {
  const int block = logical / (group_m * tiles_n);
  const int first_row = block * group_m;
  const int rows = min(group_m, tiles_m - first_row);
  const int within = logical - block * group_m * tiles_n;
  *tile_n = within / rows;
  *tile_m = first_row + within % rows;
}

// Tile rows per block for tile_of: the count that makes the `per_xcd` tiles that an XCD works on at one time read
// the fewest rows of A and W together, rows x BM + ceil(per_xcd / rows) x BN (4,096 tokens: the 7B gate/up product
// 921 to 884 us, the 72B q/k/v product 663 to 558; at 2,048 tokens, eight rows of tiles, within 2 % either way).
inline int tile_group_rows(int tiles_m, long long per_xcd, int BM, int BN) {
  int best = 1;
  long long best_cost = -1;
  for (int rows = 1; rows <= tiles_m; ++rows) {
    const long long cost = (long long)rows * BM + (per_xcd + rows - 1) / rows * BN;
    if (best_cost < 0 || cost < best_cost) {
      best = rows;
      best_cost = cost;
    }
  }
  return best;
}

// BM x BN: output tile of a workgroup (tokens x weight rows); WM x WN: its grid of waves. A wave owns
// (BM / WM) x (BN / WN) outputs as TM x TN instruction tiles.
template <int BM, int BN, int WM, int WN, typename TC, bool ACCUMULATE, bool GATED>
__global__ __launch_bounds__(WM * WN * 64) void gemm_tile_kernel(const __bf16* __restrict__ A,
                                                                   const __bf16* __restrict__ W,
                                                                   const float* __restrict__ bias, TC* __restrict__ C,
                                                                   int M, int N, int K, long long lda, long long ldc,
                                                                   int tiles_m, int tiles_n, int group_m,
                                                                   int vector_ok,
                                                                   int k_per_range, long long range_stride,
                                                                   TileNorm norm) {
  // gridDim.y > 1: K is split into ranges of k_per_range (a multiple of 64); range r writes its partial
  // sums to C + r * range_stride and a second kernel adds the ranges
  const int k_begin = blockIdx.y * k_per_range, k_end = min(K, k_begin + k_per_range);
  C += (size_t)blockIdx.y * range_stride;
  constexpr int THREADS = WM * WN * 64;
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
  constexpr int A_PIECES = BM * 8 / THREADS, W_PIECES = BN * 8 / THREADS;  // 16-byte pieces per thread and step
  static_assert(BM * 8 % THREADS == 0 && BN * 8 % THREADS == 0, "tile rows must divide among the threads");
  extern __shared__ __attribute__((aligned(16))) __bf16 lds[];
  __bf16* sA = lds;                  // [2][BM][ROW]
  __bf16* sW = lds + 2 * BM * ROW;   // [2][BN][ROW]

  // workgroups are dealt to the XCDs round-robin; give each XCD a contiguous run of tiles
  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + XCDS - 1) / XCDS;
  const int logical = (blockIdx.x % XCDS) * per_xcd + blockIdx.x / XCDS;
  if (logical >= total) return;
  int tile_m, tile_n;
  tile_of(logical, tiles_m, tiles_n, group_m, &tile_m, &tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int lr = lane & 15, lg = lane >> 4;

  f32x4 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // rows past M or N read zero through the buffer descriptors, so no load sits behind a branch
  const BufferView a_view = buffer_view(A + (size_t)m0 * lda, ((unsigned long long)(M - m0 - 1) * lda + K) * 2);
  const BufferView w_view = buffer_view(W + (size_t)n0 * K, (unsigned long long)(N - n0) * K * 2);
  unsigned a_off[A_PIECES], w_off[W_PIECES];
#pragma unroll
  for (int i = 0; i < A_PIECES; ++i) {
    const int id = tid + THREADS * i;
    a_off[i] = (unsigned)(((id >> 3) * lda + (id & 7) * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < W_PIECES; ++i) {
    const int id = tid + THREADS * i;
    w_off[i] = (unsigned)(((size_t)(id >> 3) * K + (id & 7) * 8) * 2);
  }
  bf16x8 ra[A_PIECES], rw[W_PIECES];
  auto load_global = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_PIECES; ++i) ra[i] = a_view.load(a_off[i] + (unsigned)k0 * 2);
#pragma unroll
    for (int i = 0; i < W_PIECES; ++i) rw[i] = w_view.load(w_off[i] + (unsigned)k0 * 2);
    if (k0 + BK > k_end) {  // the last step of a range that is no multiple of 64 long: pieces past its end are zero
#pragma unroll
      for (int i = 0; i < A_PIECES; ++i)
        if (k0 + ((tid + THREADS * i) & 7) * 8 >= k_end) ra[i] = zero8();
#pragma unroll
      for (int i = 0; i < W_PIECES; ++i)
        if (k0 + ((tid + THREADS * i) & 7) * 8 >= k_end) rw[i] = zero8();
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_PIECES; ++i) {
      const int id = tid + THREADS * i;
      *(bf16x8*)(sA + buf * BM * ROW + (id >> 3) * ROW + (id & 7) * 8) = ra[i];
    }
#pragma unroll
    for (int i = 0; i < W_PIECES; ++i) {
      const int id = tid + THREADS * i;
      *(bf16x8*)(sW + buf * BN * ROW + (id >> 3) * ROW + (id & 7) * 8) = rw[i];
    }
  };

  const int steps = (k_end - k_begin + BK - 1) / BK;
  __shared__ float part_sums[THREADS];
  load_global(k_begin);
  tile_norm_parts<BM, THREADS>(norm, m0, M, tid, part_sums);
  store_lds(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) load_global(k_begin + (s + 1) * BK);
    const __bf16* tA = sA + buf * BM * ROW + (wm * TM * 16 + lr) * ROW + lg * 8;
    const __bf16* tW = sW + buf * BN * ROW + (wn * TN * 16 + lr) * ROW + lg * 8;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      bf16x8 fa[TM], fw[TN];
#pragma unroll
      for (int t = 0; t < TM; ++t) fa[t] = *(const bf16x8*)(tA + t * 16 * ROW + ks * 32);
#pragma unroll
      for (int t = 0; t < TN; ++t) fw[t] = *(const bf16x8*)(tW + t * 16 * ROW + ks * 32);
#pragma unroll
      for (int tn = 0; tn < TN; ++tn)
#pragma unroll
        for (int tm = 0; tm < TM; ++tm)
          acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[tn], fa[tm], acc[tn][tm], 0, 0, 0);
    }
    if (s + 1 < steps) store_lds(buf ^ 1);
    __syncthreads();
  }

  tile_epilogue<BM, THREADS, TM, TN, TC, ACCUMULATE, GATED>(acc, C, ldc, M, N, K, bias, vector_ok != 0,
                                                            m0 + wm * TM * 16, n0 + wn * TN * 16, lr, lg, norm,
                                                            part_sums, wm * TM * 16);
}

// ---------------------------------------------------------------------------------------------
// The tiled product with both operands loaded straight into LDS (buffer loads with the lds modifier: no
// staging registers, no LDS store instructions) and a software pipeline inside each wave: two register
// sets of operand fragments, one being read from LDS while the other is multiplied, so that a wave keeps
// the matrix core busy by itself and a wave tile of 64 x 128 (eight waves per 256 x 256 tile) fits the
// register file. Per K step of 64 a CU then reads 192 KB of fragments from LDS, against 256 KB with
// sixteen waves of 64 x 64.
//
// LDS rows are 128 bytes, unpadded (a load instruction fills 1 KB: 8 rows, lane L the 16 bytes at 16 L).
// The 16-byte chunk c of row r sits in slot c ^ (r % 8); the loading lane picks the global chunk that
// belongs in its slot, the reading lane the slot of its chunk, and 16 rows read the same chunk from
// different banks.
//
// Step s works on stage s % 2, the fragments of its first half (k 0..31 of the step) already in registers:
//   read the fragments of the second half; multiply the first half;
//   wait for the own loads of step s + 1, barrier (now nobody reads stage s % 2 any more);
//   issue the loads of step s + 2 into stage s % 2; read the first-half fragments of step s + 1;
//   multiply the second half.
// K ranges must be multiples of 64 (the launcher sends other shapes to gemm_tile_kernel). Four stages of
// 32 k, which give a load three short steps to arrive instead of one long one, were slower.
// STAGES 3 (for up to 128 tokens, where the product is a stream of the weights and a CU's bytes in flight are
// what bounds it): step s + 3 is requested when step s's stage is free, and the barrier of a step waits for
// step s + 1 only, so the loads of two steps are in flight instead of one.
constexpr int DIRECT_ROW = BK * 2;  // bytes per LDS row

// Until none of the wave's vector memory loads is in flight (s_waitcnt vmcnt(0), the other counters left
// alone). A barrier alone does not wait for loads that write LDS: the compiler's fence only waits for the
// wave's LDS instructions.
__device__ __forceinline__ void wait_own_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }
// Until at most N of them are (loads complete in the order of their issue): s_waitcnt vmcnt(N).
template <int N>
__device__ __forceinline__ void wait_own_loads_but() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt((N & 15) | ((N >> 4) << 14) | 0x0F70);
}

template <int BM, int BN, int WM, int WN, typename TC, bool ACCUMULATE, bool GATED, int STAGES = 2>
__global__ __launch_bounds__(WM * WN * 64) void gemm_tile_direct_kernel(const __bf16* __restrict__ A,
                                                                          const __bf16* __restrict__ W,
                                                                          const float* __restrict__ bias,
                                                                          TC* __restrict__ C, int M, int N, int K,
                                                                          long long lda, long long ldc, int tiles_m,
                                                                          int tiles_n, int group_m, int vector_ok,
                                                                          int k_per_range,
                                                                          long long range_stride, TileNorm norm) {
  typedef __attribute__((address_space(3))) void* lds_ptr;
  const int k_begin = blockIdx.y * k_per_range, k_end = min(K, k_begin + k_per_range);
  C += (size_t)blockIdx.y * range_stride;
  constexpr int WAVES = WM * WN;
  constexpr int TM = BM / WM / 16, TN = BN / WN / 16;
  constexpr int A_LOADS = BM / 8 / WAVES, W_LOADS = BN / 8 / WAVES;  // load instructions per wave and step
  static_assert(BM % (8 * WAVES) == 0 && BN % (8 * WAVES) == 0, "tile rows must divide among the waves' loads");
  constexpr int STAGE = (BM + BN) * DIRECT_ROW;
  constexpr int LOADS = A_LOADS + W_LOADS;
  static_assert(STAGES == 2 || STAGES == 3, "two or three LDS stages");
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];  // [STAGES][BM + BN][128]

  const int total = tiles_m * tiles_n;
  const int per_xcd = (total + XCDS - 1) / XCDS;
  const int logical = (blockIdx.x % XCDS) * per_xcd + blockIdx.x / XCDS;
  if (logical >= total) return;
  int tile_m, tile_n;
  tile_of(logical, tiles_m, tiles_n, group_m, &tile_m, &tile_n);
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WN, wn = wave % WN;
  const int lr = lane & 15, lg = lane >> 4;

  f32x4 acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; ++i)
#pragma unroll
    for (int j = 0; j < TM; ++j) acc[i][j] = f32x4{0.f, 0.f, 0.f, 0.f};

  // rows past M or N read zero through the buffer descriptors
  const BufferView a_view = buffer_view(A + (size_t)m0 * lda, ((unsigned long long)(M - m0 - 1) * lda + K) * 2);
  const BufferView w_view = buffer_view(W + (size_t)n0 * K, (unsigned long long)(N - n0) * K * 2);
  // a load instruction covers 8 rows: lane L fills slot L % 8 of row L / 8 with chunk (L % 8) ^ (L / 8)
  const int ld_row = lane >> 3, ld_chunk = (lane & 7) ^ (lane >> 3);
  unsigned a_off[A_LOADS], w_off[W_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i)
    a_off[i] = (unsigned)((((wave * A_LOADS + i) * 8 + ld_row) * lda + ld_chunk * 8 + k_begin) * 2);
#pragma unroll
  for (int i = 0; i < W_LOADS; ++i)
    w_off[i] = (unsigned)((((size_t)(wave * W_LOADS + i) * 8 + ld_row) * K + ld_chunk * 8 + k_begin) * 2);
  auto issue_loads = [&](int stage, int step) {
    unsigned char* to_a = lds_raw + stage * STAGE + wave * A_LOADS * 1024;
    unsigned char* to_w = lds_raw + stage * STAGE + BM * DIRECT_ROW + wave * W_LOADS * 1024;
    const unsigned kb = (unsigned)step * (BK * 2);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(a_view.rsrc, (lds_ptr)(to_a + i * 1024), 16, (int)(a_off[i] + kb), 0, 0, 0);
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(w_view.rsrc, (lds_ptr)(to_w + i * 1024), 16, (int)(w_off[i] + kb), 0, 0, 0);
  };
  // a lane's fragment chunks within a stage: row lr of each 16-row tile, chunk lg (first half of the step)
  // or lg + 4 (second half), which differ in bit 6 of the byte offset
  const unsigned frag_a = (unsigned)((wm * TM * 16 + lr) * DIRECT_ROW + ((lg ^ (lr & 7)) * 16));
  const unsigned frag_w = (unsigned)(BM * DIRECT_ROW + (wn * TN * 16 + lr) * DIRECT_ROW + ((lg ^ (lr & 7)) * 16));
  auto read_fragments = [&](int stage, int half, bf16x8 (&fa)[TM], bf16x8 (&fw)[TN]) {
    const unsigned char* base = lds_raw + stage * STAGE;
#pragma unroll
    for (int t = 0; t < TN; ++t) fw[t] = *(const bf16x8*)(base + (frag_w ^ (half * 64)) + t * 16 * DIRECT_ROW);
#pragma unroll
    for (int t = 0; t < TM; ++t) fa[t] = *(const bf16x8*)(base + (frag_a ^ (half * 64)) + t * 16 * DIRECT_ROW);
  };
  auto multiply = [&](const bf16x8 (&fa)[TM], const bf16x8 (&fw)[TN]) {
#pragma unroll
    for (int tn = 0; tn < TN; ++tn)
#pragma unroll
      for (int tm = 0; tm < TM; ++tm)
        acc[tn][tm] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fw[tn], fa[tm], acc[tn][tm], 0, 0, 0);
  };

  const int steps = (k_end - k_begin) / BK;
  bf16x8 fa0[TM], fw0[TN], fa1[TM], fw1[TN];
  __shared__ float part_sums[WAVES * 64];
  issue_loads(0, 0);
  if (steps > 1) issue_loads(1, 1);
  if (STAGES == 3 && steps > 2) issue_loads(2, 2);
  tile_norm_parts<BM, WAVES * 64>(norm, m0, M, tid, part_sums);  // behind the first requests, before the first wait
  if (STAGES == 3 && steps > 2) {
    wait_own_loads_but<2 * LOADS>();  // step 0 has arrived; the other two stay in flight
  } else {
    wait_own_loads();
  }
  __syncthreads();
  read_fragments(0, 0, fa0, fw0);
  // Hints for the instruction order within a half step: the LDS reads and the loads go out one by one
  // between products, so that their issue hides behind the matrix core's work instead of stalling it.
  auto interleave = [](auto lds_reads, auto loads) {
    constexpr int READS = decltype(lds_reads)::value, LOADS_NOW = decltype(loads)::value;
    static_for<LOADS_NOW>([](auto) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one matrix instruction
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one load
    });
    static_for<READS>([](auto) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
    });
    __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
  };
  // `in_flight`: how many later steps' loads may stay in flight at the barrier (all of a step's loads that were
  // issued before them have then arrived)
  auto step = [&](int s, int stage, auto with_loads, auto with_next, auto in_flight) {
    const int next_stage = stage + 1 == STAGES ? 0 : stage + 1;
    read_fragments(stage, 1, fa1, fw1);
    multiply(fa0, fw0);
    interleave(std::integral_constant<int, TM + TN>{}, std::integral_constant<int, 0>{});
    __builtin_amdgcn_sched_barrier(0);  // the products stay on this side: they cover the reads above
    wait_own_loads_but<decltype(in_flight)::value * LOADS>();
    __syncthreads();
    if constexpr (decltype(with_loads)::value) issue_loads(stage, s + STAGES);
    if constexpr (decltype(with_next)::value) read_fragments(next_stage, 0, fa0, fw0);
    multiply(fa1, fw1);
    interleave(std::integral_constant<int, decltype(with_next)::value ? TM + TN : 0>{},
               std::integral_constant<int, decltype(with_loads)::value ? LOADS : 0>{});
    __builtin_amdgcn_sched_barrier(0);
  };
  int s = 0, stage = 0;
  auto advance = [&]() { stage = stage + 1 == STAGES ? 0 : stage + 1; };
  for (; s + STAGES < steps; ++s, advance())   // with three stages the step after next stays in flight
    step(s, stage, std::true_type{}, std::true_type{}, std::integral_constant<int, STAGES - 2>{});
  for (; s + 1 < steps; ++s, advance())
    step(s, stage, std::false_type{}, std::true_type{}, std::integral_constant<int, 0>{});
  step(s, stage, std::false_type{}, std::false_type{}, std::integral_constant<int, 0>{});

  tile_epilogue<BM, WAVES * 64, TM, TN, TC, ACCUMULATE, GATED>(acc, C, ldc, M, N, K, bias, vector_ok != 0,
                                                               m0 + wm * TM * 16, n0 + wn * TN * 16, lr, lg, norm,
                                                               part_sums, wm * TM * 16);
}

// ---------------------------------------------------------------------------------------------
constexpr int SPAN = 128;  // k per wave per step: four instructions of 32

// The K loop of the weight-streaming kernels: wave `wave` of WAVES multiplies the spans wave, wave + WAVES, ...
// of K (and the rest of K, less than a span, falls to one of them) into acc. w_off / a_off: a lane's byte offsets
// of its operand rows at k = 0. `between` runs once the first spans are requested and before the first product:
// work that waits for earlier loads costs nothing there, the weights are on their way meanwhile.
struct Nothing {
  __device__ __forceinline__ void operator()() const {}
};
template <int CB, int RT, int WAVES, int SETS, typename Between = Nothing>
__device__ __forceinline__ void skinny_products(const BufferView& w_view, const BufferView& a_view,
                                                const unsigned (&w_off)[RT], const unsigned (&a_off)[CB], int K, int wave,
                                                int lg, f32x4 (&acc)[RT][CB], Between between = Between()) {
  // SETS register sets of operands rotate through run_pipeline: the loads of SETS - 1 spans are in flight
  // while one span is multiplied (three sets with one block of tokens, two with more).
  bf16x8 wf[SETS][RT][4], af[SETS][CB][4];
  auto load_span = [&](int span, bf16x8 (&w_dst)[RT][4], bf16x8 (&a_dst)[CB][4]) {
    const unsigned kb = (unsigned)span * SPAN * 2;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) w_dst[rt][i] = w_view.load(w_off[rt] + kb + i * 64);
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) a_dst[cb][i] = a_view.load(a_off[cb] + kb + i * 64);
    }
  };
  auto multiply = [&](const bf16x8 (&w_src)[RT][4], const bf16x8 (&a_src)[CB][4]) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w_src[rt][i], a_src[cb][i], acc[rt][cb], 0, 0, 0);
  };
  const int whole = K / SPAN;                                               // spans that lie inside K
  const int count = wave < whole ? (whole - wave + WAVES - 1) / WAVES : 0;  // this wave's: wave + i * WAVES
  auto step = [&](auto set_, auto rem_, int i) {
    constexpr int SET = decltype(set_)::value;
    if constexpr (decltype(rem_)::value >= SETS - 1)
      load_span(wave + (i + SETS - 1) * WAVES, wf[(SET + SETS - 1) % SETS], af[(SET + SETS - 1) % SETS]);
    multiply(wf[SET], af[SET]);
  };
  if (count >= SETS - 1) {
    static_for<SETS - 1>([&](auto j) { load_span(wave + j.value * WAVES, wf[j.value], af[j.value]); });
    between();
    run_pipeline<SETS, SETS - 1>(step, count);
  } else {  // fewer spans than the pipeline is deep: request them all, then multiply
    static_for<SETS - 1>([&](auto j) {
      if (j.value < count) load_span(wave + j.value * WAVES, wf[j.value], af[j.value]);
    });
    between();
    static_for<SETS - 1>([&](auto j) {
      if (j.value < count) multiply(wf[j.value], af[j.value]);
    });
  }
  if (whole * SPAN < K && wave == whole % WAVES) {  // the rest of K, less than a span: operands past K are zeroed
    load_span(whole, wf[0], af[0]);
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (whole * SPAN + i * 32 + lg * 8 >= K) {
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) wf[0][rt][i] = zero8();
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) af[0][cb][i] = zero8();
      }
    multiply(wf[0], af[0]);
  }
}

// CB: blocks of 16 tokens (M <= 16 * CB). RT: tiles of 16 weight rows per wave. WAVES: waves of a
// workgroup, which split K in interleaved spans. A workgroup owns 16 * RT weight rows.
// What the product that adds into the residual leaves for the RMS norm that follows it (FOLLOW): beside the new
// residual x, scaled[m][n] = bfloat16(x * gain[n]) and sumsq[workgroup][m] = the sum of x^2 over the workgroup's
// columns, 16 floats per workgroup. The product after the norm adds the workgroups' sums in a fixed order, takes
// 1 / sqrt(mean + eps) and scales its own 32-bit sums with it: the norm costs no launch and no workgroup waits
// for a whole row (crates/vipera-backend-cpu/src/model.rs:4282-4288 is the formula; the rounding to bfloat16 falls
// on x * gain instead of x * inv * gain).
struct FollowNorm {
  const float* gain;
  __bf16* scaled;
  float* sumsq;
  long long ld_scaled;
  int sumsq_stride = 16;  // floats per workgroup: 16 tokens for the consumers of up to 16 tokens, 64 beyond
};

// The consumer's side of FollowNorm in a workgroup of 256 threads. request_squares: thread t asks for the sums of
// groups t and t + 256 (at most 512 groups), unconditionally at clamped addresses, because a load behind a branch
// would make the compiler wait for every load in flight; call it before the kernel's other loads. add_squares: the
// 16 tokens' sums over the wave's lanes with 17 exchanges (at each of four steps a lane keeps one half of its
// values and adds the partner's copy of that half, the lane bit choosing which; then two full steps), left in
// wave_sums[wave * 16 + token]; every index is a compile-time constant, so the values stay in registers.
// inv_rms: after a barrier, 1 / sqrt(mean + eps) of a token from the four waves' sums (a fixed order throughout).
struct Squares {
  f32x4 first[4], second[4];
};
__device__ __forceinline__ Squares request_squares(const float* __restrict__ sumsq, int groups, int tid) {
  Squares q;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    q.first[i] = *(const f32x4*)(sumsq + (size_t)min(tid, groups - 1) * 16 + i * 4);
    q.second[i] = *(const f32x4*)(sumsq + (size_t)min(tid + 256, groups - 1) * 16 + i * 4);
  }
  return q;
}
__device__ __forceinline__ void add_squares(const Squares& q, int groups, int tid, float* wave_sums) {
  const int lane = tid & 63, wave = tid >> 6;
  const bool has = tid < groups, has_more = tid + 256 < groups;
  float v[16];
#pragma unroll
  for (int m = 0; m < 16; ++m) v[m] = (has ? q.first[m / 4][m % 4] : 0.f) + (has_more ? q.second[m / 4][m % 4] : 0.f);
  static_for<4>([&](auto step) {
    constexpr int bit = 1 << step.value, n = 8 >> step.value;
    const bool upper = (lane & bit) != 0;
    static_for<n>([&](auto i) {
      const float got = __shfl_xor(upper ? v[i.value] : v[i.value + n], bit);
      v[i.value] = (upper ? v[i.value + n] : v[i.value]) + got;
    });
  });
  v[0] += __shfl_xor(v[0], 16);
  v[0] += __shfl_xor(v[0], 32);
  if (lane < 16) wave_sums[wave * 16 + ((lane & 1) * 8 + (lane & 2) * 2 + (lane & 4) / 2 + (lane & 8) / 8)] = v[0];
}
__device__ __forceinline__ float inv_rms(const float* wave_sums, int token, int width, float eps) {
  const float sum = wave_sums[token] + wave_sums[16 + token] + wave_sums[32 + token] + wave_sums[48 + token];
  return 1.0f / sqrtf(sum / (float)width + eps);
}

template <int CB, int RT, int WAVES, typename TC, bool ACCUMULATE, int SETS = (CB == 1 ? VK_SKINNY_SETS : 2),
          bool FOLLOW = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const __bf16* __restrict__ A,
                                                                  const __bf16* __restrict__ W,
                                                                  const float* __restrict__ bias,
                                                                  TC* __restrict__ C, int M, int N, int K,
                                                                  long long lda, long long ldc, int vector_ok,
                                                                  int rows, FollowNorm follow) {
  static_assert(!FOLLOW || (CB == 1 && RT == 1 && ACCUMULATE && sizeof(TC) == 4), "the norm follows a residual product");
  __shared__ f32x4 partial[WAVES][RT * CB][64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  // The workgroup owns weight rows [n0, n_end): `rows` of them, at most 16 * RT. Fewer than a full tile lets
  // the launch cut N into as many equal workgroups as fill the CUs evenly; the instruction's other rows
  // lie past the view's end.
  const int n0 = blockIdx.x * rows, n_end = min(N, n0 + rows);
  const int align = !vector_ok ? 1 : (n0 & 3) == 0 ? 4 : (n0 & 1) == 0 ? 2 : 1;
  vector_ok = align == 4;
  // reads past the workgroup's last weight row or the last token return zero and fetch nothing (see BufferView)
  const BufferView w_view = buffer_view(W + (size_t)n0 * K, (unsigned long long)(n_end - n0) * K * 2);
  const BufferView a_view = buffer_view(A, ((unsigned long long)(M - 1) * lda + K) * 2);
  unsigned w_off[RT], a_off[CB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) w_off[rt] = (unsigned)(((rt * 16 + lr) * K + lg * 8) * 2);
#pragma unroll
  for (int cb = 0; cb < CB; ++cb) a_off[cb] = (unsigned)(((cb * 16 + lr) * lda + lg * 8) * 2);
  f32x4 acc[RT][CB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) acc[rt][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

  // What the epilogue adds to the first tile this wave will store (bias, and the old C when accumulating) is
  // requested now: read after the last product it would be one more round trip to memory at the end of a
  // kernel that takes a few of them in all. Clamped addresses, so the loads are unconditional.
  f32x4 early_bias = {0.f, 0.f, 0.f, 0.f}, early_c = {0.f, 0.f, 0.f, 0.f}, early_gain = {0.f, 0.f, 0.f, 0.f};
  const bool early = vector_ok && wave < RT * CB && n_end - n0 >= 4;
  const int early_m = (wave % CB) * 16 + lr, early_n = n0 + (wave / CB) * 16 + lg * 4;
  if (early) {
    const int m = min(early_m, M - 1), n = min(early_n, n_end - 4);
    if (bias) early_bias = *(const f32x4*)(bias + n);
    if constexpr (ACCUMULATE) early_c = *(const f32x4*)((const float*)C + (size_t)m * ldc + n);
    if constexpr (FOLLOW) early_gain = *(const f32x4*)(follow.gain + n);
  }

  skinny_products<CB, RT, WAVES, SETS>(w_view, a_view, w_off, a_off, K, wave, lg, acc);
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
    if constexpr (FOLLOW) {  // one tile, wave 0: the new residual, its gained bfloat16 copy, its squares
      float squares = 0.f;
      if (lr < M) {
        if (early && early_n + 3 < n_end) {
          if (bias) sum += early_bias;
          sum += early_c;
          *(f32x4*)((float*)C + (size_t)lr * ldc + early_n) = sum;
          bf16x4 o;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            o[j] = (__bf16)(sum[j] * early_gain[j]);
            squares += sum[j] * sum[j];
          }
          *(bf16x4*)(follow.scaled + (size_t)lr * follow.ld_scaled + early_n) = o;
        } else {
          const int n = n0 + lg * 4;
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (n + j < n_end) {
              float* at = (float*)C + (size_t)lr * ldc + n + j;
              const float x = sum[j] + (bias ? bias[n + j] : 0.f) + *at;
              *at = x;
              follow.scaled[(size_t)lr * follow.ld_scaled + n + j] = (__bf16)(x * follow.gain[n + j]);
              squares += x * x;
            }
        }
      }
      squares += __shfl_xor(squares, 16);
      squares += __shfl_xor(squares, 32);
      if (lg == 0) follow.sumsq[(size_t)blockIdx.x * 16 + lr] = squares;
      continue;
    }
    if (early && t == wave && early_m < M && early_n + 3 < n_end) {
      // the same sums in the same order as store4, with the operands read at the start
      if (bias) sum += early_bias;
      TC* dst = C + (size_t)early_m * ldc + early_n;
      if constexpr (sizeof(TC) == 4) {
        if (ACCUMULATE) sum += early_c;
        *(f32x4*)dst = sum;
      } else {
        bf16x4 o;
#pragma unroll
        for (int j = 0; j < 4; ++j) o[j] = (__bf16)sum[j];
        *(bf16x4*)dst = o;
      }
      continue;
    }
    store4_aligned<TC, ACCUMULATE>(C, ldc, cb * 16 + lr, n0 + rt * 16 + lg * 4, M, n_end, sum, bias, align);
  }
}

// CUs of the current device (asked once).
int compute_units() {
  static int cus = 0;
  if (!cus) {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess)
      count = 0;
    cus = count > 0 ? count : 256;
  }
  return cus;
}

// Weight rows per tile, 8 to 16 and even (outputs go out in pairs at least), for a launch of
// `ranges` x ceil(N / (tiles * rows)) workgroups with `tiles` tiles each. A CU's time goes with the bytes it
// pulls: the rounds of workgroups over the CUs (whole rounds while they are few; with three or more the
// dispatcher evens them out) times a workgroup's rows, the activations counted as half a row per token (they
// come from L2) and eight rows for what a workgroup costs before and after its stream. Fitted to sweeps of the
// 7B and 32B products at 8 to 64 tokens. N = 3584 on 256 CUs: 256 workgroups of 14 rows instead of 224 of 16.
int balanced_rows(int M, int N, int tiles, int ranges) {
  const int cus = compute_units();
  int best = 16;
  double best_cost = 0.0;
  for (int rows = 16; rows >= 8; rows -= 2) {
    const long long groups = (long long)((N + tiles * rows - 1) / (tiles * rows)) * ranges;
    const double rounds = groups >= 3 * cus ? (double)groups / cus : (double)((groups + cus - 1) / cus);
    const double cost = rounds * (tiles * rows + 0.5 * M + 8.0);
    if (rows == 16 || cost < best_cost * 0.97) {
      best = rows;
      best_cost = cost;
    }
  }
  return best;
}

template <int CB, int RT, int WAVES, typename TC, bool ACC>
int launch_skinny_as(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                     long long ldc, int vector_ok, int rows, hipStream_t s) {
  if (rows <= 0 || rows > 16 * RT) rows = RT == 1 ? balanced_rows(M, N, 1, 1) : 16 * RT;
  const int blocks = (N + rows - 1) / rows;
  gemm_skinny_kernel<CB, RT, WAVES, TC, ACC><<<blocks, WAVES * 64, 0, s>>>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, rows,
                                                                           FollowNorm{});
  VK_LAUNCH_CHECK();
  return 0;
}

// Shape of the launch (rows per wave, waves that split K). Measured on the 7B shapes: with one block of
// tokens four waves on 16 rows are fastest at every weight size; with more blocks, many rows want two
// row tiles per wave so that activations are re-read less.
template <int CB, typename TC, bool ACC>
int launch_skinny_cb(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                     long long ldc, int vector_ok, int shape, hipStream_t s) {
  const int tiles = (N + 15) / 16;
  if (shape == 0) shape = (CB >= 2 && tiles >= 1024) ? 2 : 1;
  switch (shape) {
    case 1: return launch_skinny_as<CB, 1, 4, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, 0, s);
    case 2: return launch_skinny_as<CB, 2, 4, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, 0, s);
  }
  if (shape >= 108 && shape <= 116)  // one tile per wave with a forced number of rows per workgroup
    return launch_skinny_as<CB, 1, 4, TC, ACC>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, shape - 100, s);
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

// ---------------------------------------------------------------------------------------------
// The q/k/v product of up to 16 tokens with the rotation and the cache write in its epilogue, which saves the
// launch between the product and the attention of a decode step. The streaming is gemm_skinny_kernel's (four
// waves split K). A workgroup's tile holds `pairs` (at most 8) rotation pairs of the q and k heads, taken from the
// list of all (head, dim below half the head width): the dims in the tile's rows 0-7 and their partners half a head
// further on in rows 8-15, so a lane finds a dim's partner in lane ^ 32. Its `values` (at most 16) dims of the v
// heads sit in the rows that the pairs leave free, or, where those are too few, in a second tile (RT 2). The
// launcher picks the two numbers so that the workgroups fill the CUs evenly (28 + 4 heads of 128 and 4 v heads: 256
// workgroups of 8 pairs and, in a second tile, 2 values, 18 weight rows each; 40 + 8 and 8 heads: 512 workgroups of
// 6 pairs and 2 values in one tile; a tile's unused rows lie past the end of the buffer view and fetch nothing, but
// every load instruction costs the same, which is why one tile is preferred). The sums take
// the bias, are rounded to bfloat16 as the product alone would leave them, and are then rotated and stored exactly
// as rope_kvwrite_kernel does (crates/vipera-backend-cpu/src/model.rs:4192-4251, 1495-1542): what the cache and
// the attention see does not depend on which of the two paths a token took. Full rotation only (rotary width =
// head width).
struct QkvRope {
  const int* positions;
  const float* inv_freq;
  __bf16* k_cache;  // null: rotate only (a layer that reads another layer's cache)
  __bf16* v_cache;
  const int* entry_of_token;
  const int* block_table;
  int table_width, block_size, heads, kv_heads, hd, pairs, values;
  const float* sumsq;  // SCALED: A is x * gain of the norm before (see FollowNorm), `groups` sums of squares, `eps`
  int groups;
  float eps;
};

template <int RT, bool SCALED>
__global__ __launch_bounds__(256) void gemm_qkv_rope_kernel(const __bf16* __restrict__ A, const __bf16* __restrict__ W,
                                                            const float* __restrict__ bias, __bf16* __restrict__ C,
                                                            int M, int N, int K, long long lda, long long ldc, QkvRope r) {
  constexpr int WAVES = 4;
  constexpr unsigned NO_ROW = 0x80000000u;  // past the end of the weight's view (the launcher checks its size)
  __shared__ f32x4 partial[WAVES][RT][64];
  __shared__ float wave_sums[64];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  Squares squares;
  if constexpr (SCALED) squares = request_squares(r.sumsq, r.groups, tid);
  const int hd = r.hd, half = hd / 2;
  const int all_pairs = (r.heads + r.kv_heads) * half, all_values = r.kv_heads * hd, first_value_row = (r.heads + r.kv_heads) * hd;
  // Row i of the first tile -> its output column, or -1: slots 0 .. pairs - 1 of each half of the tile hold the
  // pairs (head * hd + dim, the partner in the other half); with one tile (RT 1) the slots behind them hold
  // the workgroup's values, the first 8 - pairs in rows pairs .. 7, the rest in rows 8 + pairs .. 15.
  auto value_of = [&](int index) {  // the workgroup's value number `index` -> column, or -1
    const int v = blockIdx.x * r.values + index;
    return index < r.values && v < all_values ? first_value_row + v : -1;
  };
  auto first_tile_column = [&](int i, bool& rotated) {
    const int slot = i & 7, pair = blockIdx.x * r.pairs + slot;
    rotated = slot < r.pairs;
    if (rotated) return pair < all_pairs ? (pair / half) * hd + pair % half + (i >= 8 ? half : 0) : -1;
    return RT == 1 ? value_of(slot - r.pairs + (i >= 8 ? 8 - r.pairs : 0)) : -1;
  };
  const BufferView w_view = buffer_view(W, (unsigned long long)N * K * 2);
  const BufferView a_view = buffer_view(A, ((unsigned long long)(M - 1) * lda + K) * 2);
  unsigned w_off[RT];
  {
    bool unused;
    const int row0 = first_tile_column(lr, unused);
    w_off[0] = row0 >= 0 ? (unsigned)(((size_t)row0 * K + lg * 8) * 2) : NO_ROW;
    if constexpr (RT == 2) {
      const int row1 = value_of(lr);
      w_off[1] = row1 >= 0 ? (unsigned)(((size_t)row1 * K + lg * 8) * 2) : NO_ROW;
    }
  }
  const unsigned a_off[1] = {(unsigned)((lr * lda + lg * 8) * 2)};
  // What the epilogue needs from memory is requested now (clamped, so the loads are unconditional). Wave 0 finishes
  // the first tile, wave 1 the second.
  const int token = min(lr, M - 1);
  const int pos = r.positions[token];
  const int entry = r.k_cache ? r.entry_of_token[token] : 0;
  int column[4];
  bool rotated[4];
  float b[4], freq[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    rotated[j] = false;
    column[j] = wave == 0 ? first_tile_column(lg * 4 + j, rotated[j]) : value_of(lg * 4 + j);
    b[j] = bias ? bias[max(column[j], 0)] : 0.f;
    freq[j] = r.inv_freq[rotated[j] ? max(column[j], 0) % hd % half : 0];
  }

  f32x4 acc[RT][1];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) acc[rt][0] = f32x4{0.f, 0.f, 0.f, 0.f};
  // the page id and the sines wait for the position, which was requested before the weights: they are worked out
  // while the first weights are on their way, not between the last product and the stores
  int page = -1;
  float sn[4], cs[4];
  auto lookups = [&]() {
    if constexpr (SCALED) add_squares(squares, r.groups, tid, wave_sums);
    if (r.k_cache) page = r.block_table[(size_t)entry * r.table_width + pos / r.block_size];
#pragma unroll
    for (int j = 0; j < 4; ++j) sincosf((float)pos * freq[j], &sn[j], &cs[j]);
  };
  skinny_products<1, RT, WAVES, VK_SKINNY_SETS>(w_view, a_view, w_off, a_off, K, wave, lg, acc, lookups);
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) partial[wave][rt][lane] = acc[rt][0];
  __syncthreads();
  if (wave >= RT) return;
  f32x4 sum = partial[0][wave][lane];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) sum += partial[w][wave][lane];
  const int slot = pos % r.block_size;
  if constexpr (SCALED) sum *= inv_rms(wave_sums, token, K, r.eps);  // the barrier above has published the waves' sums
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float x = (float)(__bf16)(sum[j] + b[j]);
    const float y = __shfl_xor(x, 32);  // in the first tile: the partner dim's value of the same token
    __bf16 out = (__bf16)x;
    if (rotated[j]) {
      const float lo = lg < 2 ? x : y, hi = lg < 2 ? y : x;
      out = (__bf16)(lg < 2 ? lo * cs[j] - hi * sn[j] : lo * sn[j] + hi * cs[j]);
    }
    if (lr < M && column[j] >= 0) {
      C[(size_t)lr * ldc + column[j]] = out;
      if (page < 0) continue;
      if (rotated[j]) {
        const int kvh = column[j] / hd - r.heads;
        if (kvh >= 0) r.k_cache[(((size_t)page * r.kv_heads + kvh) * r.block_size + slot) * hd + column[j] % hd] = out;
      } else {
        const int v = column[j] - first_value_row;
        r.v_cache[(((size_t)page * r.kv_heads + v / hd) * hd + v % hd) * r.block_size + slot] = out;
      }
    }
  }
}

// Pairs and values per workgroup of gemm_qkv_rope_kernel: as in balanced_rows, the workgroups' rounds over the CUs
// times a workgroup's rows, tokens and fixed cost.
void qkv_rope_plan(int M, int heads, int kv_heads, int hd, int* pairs, int* values, int* groups) {
  const int cus = compute_units();
  const int all_pairs = (heads + kv_heads) * (hd / 2), all_values = kv_heads * hd;
  double best_cost = 0.0;
  for (int p = 8; p >= 4; --p) {
    const int by_pairs = (all_pairs + p - 1) / p, by_values = (all_values + 15) / 16;
    const int g = by_pairs > by_values ? by_pairs : by_values;
    const int v = (all_values + g - 1) / g;
    const double rounds = g >= 3 * cus ? (double)g / cus : (double)((g + cus - 1) / cus);
    const int tiles = v <= 2 * (8 - p) ? 1 : 2;
    const double cost = rounds * (2 * p + v + 0.5 * M + 8.0 + 2.0 * (tiles - 1));
    if (p == 8 || cost < best_cost * 0.97) {
      best_cost = cost;
      *pairs = p;
      *values = v;
      *groups = g;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// M <= 128, activations shared through LDS. A workgroup owns 64 * RT weight rows (16 * RT per wave; with
// RT 1 the launcher may give a wave fewer rows, see balanced_rows) and a range of K; all four waves walk that range together in chunks of 256. A chunk's activations
// (16 * CB tokens x 256) are fetched once per workgroup into LDS, double-buffered, one barrier per
// chunk; the weights go from HBM straight into the instruction's operand layout, the next chunk's
// loads in flight while the current one is multiplied. With several K ranges (gridDim.y > 1) every
// range writes its partial sums, [range, M, N] floats, and gemm_reduce_kernel adds the ranges in
// ascending order afterwards (a second launch: kernel boundaries are what keeps the XCDs' caches coherent).
constexpr int MID_CHUNK = 256;
constexpr int MID_ROW = MID_CHUNK + 8;  // elements per LDS row: 528 bytes, so 16 rows hit 16 different 16-byte slots
// More than four blocks of 16 tokens walk K in chunks of 128, so that two workgroups' buffers still share a CU's LDS.
constexpr int mid_chunk(int cb) { return cb > 4 ? 128 : MID_CHUNK; }

template <int CB, int RT, typename TC, bool ACCUMULATE, bool GATED = false,
          int SETS = (RT == 1 && CB <= 2 ? VK_MID_SETS : 2), int CHUNK = mid_chunk(CB)>
__global__ __launch_bounds__(256) void gemm_mid_kernel(const __bf16* __restrict__ A, const __bf16* __restrict__ W,
                                                       const float* __restrict__ bias, TC* __restrict__ C, int M,
                                                       int N, int K, long long lda, long long ldc, int k_per_range,
                                                       long long range_stride, int vector_ok, int rows) {
  extern __shared__ __attribute__((aligned(16))) __bf16 lds[];  // [2][CB * 16][ROW]
  constexpr int ROW = CHUNK + 8, PIECES = CHUNK / 8, KSTEPS = CHUNK / 32;
  constexpr int BUF = CB * 16 * ROW;
  constexpr int A_LOADS = CB * 16 * PIECES / 256;  // 16-byte pieces of a chunk per thread
  static_assert(CB * 16 * PIECES % 256 == 0, "a chunk's pieces must divide among the threads");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  // a wave owns weight rows [n0, n_end): `rows` of them, at most 16 * RT (fewer than the tiles hold lets the
  // launch cut N into as many equal workgroups as fill the CUs evenly; the other rows lie past the view's end)
  const int n0 = (blockIdx.x * 4 + wave) * rows, n_end = min(N, n0 + rows);
  const int k_begin = blockIdx.y * k_per_range, k_end = min(K, k_begin + k_per_range);
  C += (size_t)blockIdx.y * range_stride;

  // Reads go through buffer descriptors: one past the end (a weight row past N, a token past M) returns
  // zero and fetches nothing, so no load of the pipeline below sits behind a branch, the compiler can
  // count exactly which loads a use waits for, and the later ones stay in flight.
  const BufferView w_view = buffer_view(W + (size_t)min(n0, N - 1) * K, n0 < N ? (unsigned long long)(n_end - n0) * K * 2 : 0);
  const BufferView a_view = buffer_view(A, ((unsigned long long)(M - 1) * lda + K) * 2);
  unsigned w_off[RT], a_off[A_LOADS];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) w_off[rt] = (unsigned)(((rt * 16 + lr) * K + lg * 8) * 2);
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int id = tid + 256 * i;
    a_off[i] = (unsigned)(((id / PIECES) * lda + (id % PIECES) * 8) * 2);
  }
  f32x4 acc[RT][CB];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int cb = 0; cb < CB; ++cb) acc[rt][cb] = f32x4{0.f, 0.f, 0.f, 0.f};

  bf16x8 a_stage[A_LOADS], w[SETS][RT][KSTEPS];
  auto load_acts = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) a_stage[i] = a_view.load(a_off[i] + (unsigned)k0 * 2);
  };
  auto store_acts = [&](int buf) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int id = tid + 256 * i;
      *(bf16x8*)(lds + buf * BUF + (id / PIECES) * ROW + (id % PIECES) * 8) = a_stage[i];
    }
  };
  auto load_weights = [&](int k0, bf16x8 (&dst)[RT][KSTEPS]) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < KSTEPS; ++i) dst[rt][i] = w_view.load(w_off[rt] + (unsigned)(k0 + i * 32) * 2);
  };
  auto multiply = [&](const bf16x8 (&wf)[RT][KSTEPS], int buf) {
    const __bf16* tile = lds + buf * BUF + lr * ROW + lg * 8;
#pragma unroll
    for (int i = 0; i < KSTEPS; ++i)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb) {
        const bf16x8 a = *(const bf16x8*)(tile + cb * 16 * ROW + i * 32);
#pragma unroll
        for (int rt = 0; rt < RT; ++rt)
          acc[rt][cb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][i], a, acc[rt][cb], 0, 0, 0);
      }
  };

  // Whole chunks run through run_pipeline: the weights of chunk c + SETS - 1 are requested before chunk c
  // is multiplied (SETS register sets: three while registers allow three waves a SIMD, else two), the activations
  // of chunk c + 1 wait in registers until the barrier frees their LDS buffer, those of chunk c + 2 are
  // requested right after it.
  // Where the weight's rows lie a multiple of 4 KB apart, the range's chunks are taken in a rotated order, chunk
  // (c + turn) % whole at place c, with a turn of its own for each of the workgroups that share an XCD (every
  // eighth): workgroups with equal shares walk K in step, and with such a K all rows of the weight put the same
  // chunk on the same memory channels (8,192 x 8,192 at 8 tokens: 35.5 us without the turn, between 25.3 us at
  // K = 7,680 and 28.3 at 8,704; 25.2 with it). Not otherwise: other row lengths showed no such loss, and in
  // step the workgroups of an XCD read the same activations at the same time, out of L2.
  const int whole = (k_end - k_begin) / CHUNK;
  const bool turned = whole > 0 && (K & 2047) == 0;
  const int turn = turned ? (int)((blockIdx.x + blockIdx.y * gridDim.x) >> 3) % whole : 0;
  auto k_at = [&](int c) {  // c up to the pipeline's depth past the range: such requests read what is not used
    int j = c + turn;
    if (j >= whole) j -= whole;
    return k_begin + j * CHUNK;
  };
  int buf = 0;
  constexpr int NEED = SETS - 1 > 2 ? SETS - 1 : 2;
  auto chunk = [&](auto set_, auto rem_, int c) {
    constexpr int SET = decltype(set_)::value, REM = decltype(rem_)::value;  // REM chunks follow (capped)
    if constexpr (REM >= SETS - 1) load_weights(k_at(c + SETS - 1), w[(SET + SETS - 1) % SETS]);
    multiply(w[SET], buf);
    if constexpr (REM >= 1) store_acts(buf ^ 1);
    __syncthreads();
    if constexpr (REM >= 2) load_acts(k_at(c + 2));
    buf ^= 1;
  };
  if (whole > 0) {
    // requests past the range (fewer chunks than the pipeline is deep) read weights that are not used
    load_acts(k_at(0));
    static_for<SETS - 1>([&](auto j) { load_weights(k_at(j.value), w[j.value]); });
    store_acts(0);
    load_acts(k_at(1));
    __syncthreads();
    run_pipeline<SETS, NEED>(chunk, whole);
  }
  // the rest of the range (less than a chunk): operands past k_end are zeroed
  const int k_rest = k_begin + whole * CHUNK;
  if (k_rest < k_end) {
    load_acts(k_rest);
    load_weights(k_rest, w[0]);
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      if (k_rest + ((tid + 256 * i) % PIECES) * 8 >= k_end) a_stage[i] = zero8();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int i = 0; i < KSTEPS; ++i)
        if (k_rest + i * 32 + lg * 8 >= k_end) w[0][rt][i] = zero8();
    store_acts(0);
    __syncthreads();
    multiply(w[0], 0);
    __syncthreads();  // the epilogue may reuse the buffers
  }
  if constexpr (GATED) {
    if constexpr (RT == 2) {  // a wave's two tiles are the gate and up rows of the same outputs
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
        store_gated((__bf16*)C, ldc, cb * 16 + lr, n0 / 2 + lg * 4, M, N / 2, acc[0][cb], acc[1][cb]);
    } else {  // waves 0 and 2 hold gate rows, waves 1 and 3 the up rows of the same outputs: hand them over in LDS
      f32x4* swap = (f32x4*)lds;  // the loop's last barrier has passed: the activation buffers are free
      if (wave & 1) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb) swap[((wave >> 1) * CB + cb) * 64 + lane] = acc[0][cb];
      }
      __syncthreads();
      if (!(wave & 1)) {
#pragma unroll
        for (int cb = 0; cb < CB; ++cb)
          store_gated((__bf16*)C, ldc, cb * 16 + lr, n0 / 2 + lg * 4, M, N / 2, acc[0][cb],
                      swap[((wave >> 1) * CB + cb) * 64 + lane]);
      }
    }
  } else {
    const int align = !vector_ok ? 1 : (n0 & 3) == 0 ? 4 : (n0 & 1) == 0 ? 2 : 1;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int cb = 0; cb < CB; ++cb)
        store4_aligned<TC, ACCUMULATE>(C, ldc, cb * 16 + lr, n0 + rt * 16 + lg * 4, M, n_end, acc[rt][cb], bias, align);
  }
}

// ---------------------------------------------------------------------------------------------
// The gated product of up to 16 tokens with the activations resident in LDS. The launch has one workgroup
// per CU (its LDS request keeps a second one away) and cuts the outputs into as many contiguous runs of a multiple
// of four, so every CU pulls the same number of bytes to within four gate and four up rows: with a
// fixed tile per workgroup the CUs that get one workgroup more than the others set the time, and with runs of
// whole pairs of 16 gate and 16 up rows the busiest CU still had 8 % more than the mean at the 7B width (4 or 5
// pairs) and 37 % at the 1.5B width (2 or 3). A run's pairs are its own: pair p of a run holds the outputs
// begin + 16 p .. + 15, whichever rows of the weight those are (a lane's row is that of its output, and the rows of
// two neighbouring pairs of the weight lie 32 apart whatever the output), and in a run's last pair the lanes past
// its end request nothing. A workgroup
// copies the activations into LDS once (all of K), and from then on its four waves do not meet: the run's
// (pair, chunk of 256 k) units are cut into four equal stretches, a wave streams its stretch of weights
// from HBM straight into operand registers, SETS register sets deep (two, three and four measured the
// same), across pair boundaries without draining. Where a stretch begins or ends inside a pair the wave leaves its partial sums in LDS, and the
// wave that holds the pair's first unit adds the parts in wave order: the order of the sums depends on N,
// K and the number of workgroups only. K must be a multiple of 128: chunks of 256, or of 128 where 256 does not
// divide K (a width of 896).
#ifndef VK_RESIDENT_SETS
#define VK_RESIDENT_SETS 3
#endif
constexpr int RES_PARTIAL_BYTES = 4 * 2 * 2 * 64 * 16;  // [wave][first or last pair of its stretch][gate, up][lane]
constexpr int RES_NORM_BYTES = 4 * 16 * 4;               // [wave][token]: sums of squares (SCALED)
constexpr int RES_HEAD_BYTES = RES_PARTIAL_BYTES + RES_NORM_BYTES;

// SCALED: the activations are x * gain of a norm whose division is still to come (see FollowNorm): the sums of
// squares of `groups` workgroups, 16 floats each, are added here in a fixed order (a thread takes every 256th
// workgroup, then the block's tree), and 1 / sqrt(mean + eps) scales gate and up before the activation.
template <int SETS, bool SCALED, int RES_CHUNK = 256>
__global__ __launch_bounds__(256) void gemm_resident_gated_kernel(const __bf16* __restrict__ A,
                                                                  const __bf16* __restrict__ W,
                                                                  __bf16* __restrict__ C, int M, int N, int K,
                                                                  long long lda, long long ldc,
                                                                  const float* __restrict__ sumsq, int groups, float eps) {
  extern __shared__ __attribute__((aligned(16))) unsigned char res_lds[];
  f32x4* partial = (f32x4*)res_lds;
  float* norm_part = (float*)(res_lds + RES_PARTIAL_BYTES);
  __bf16* acts = (__bf16*)(res_lds + RES_HEAD_BYTES);  // [M][K + 8]: 16 rows start in 16 different 16-byte slots
  const int row_elems = K + 8;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lr = lane & 15, lg = lane >> 4;
  const int chunks = K / RES_CHUNK, quads = N / 8;   // N / 2 outputs, four at a time
  const int o_begin = (int)((long long)quads * blockIdx.x / gridDim.x) * 4;
  const int o_end = (int)((long long)quads * (blockIdx.x + 1) / gridDim.x) * 4;
  const int run_pairs = (o_end - o_begin + 15) / 16;
  const int last_rows = o_end - o_begin - 16 * (run_pairs - 1);   // outputs of the run's last pair
  const int units = run_pairs * chunks;
  auto bound = [&](int w) { return (int)((long long)units * w / 4); };
  const int u0 = bound(wave), u1 = bound(wave + 1), count = u1 - u0;
  const int first_pair = u0 / chunks, first_chunk = u0 % chunks;  // within the workgroup's run

  // the lane's output in the wave's first pair, and its gate row in the weight (the up row lies 16 further on)
  const int o_first = o_begin + 16 * first_pair;
  const int o_lane = o_first + lr;
  const size_t w_first_row = (size_t)(o_first / 16) * 32;           // the first row any lane of the wave needs
  const int row_lane = (o_lane / 16) * 32 + o_lane % 16 - (int)w_first_row;
  const BufferView w_view = buffer_view(W + w_first_row * K, (unsigned long long)(N - w_first_row) * K * 2);
  unsigned w_off[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) w_off[rt] = (unsigned)(((size_t)(rt * 16 + row_lane) * K + lg * 8) * 2);
  // Where the weight's rows lie a multiple of 4 KB apart, a pair's chunks are taken in a rotated order, chunk
  // (c + turn) % chunks at place c, with a turn of its own for each of the workgroups that share an XCD (every
  // eighth): runs of equal length move through their pairs in step, and with such a K all rows of the weight put
  // the same chunk on the same memory channels (the 3B width, 2,048: 26.3 us without the turn, between 18.7 us
  // at K = 1,792 and 23.3 at 2,304; 22.4 with it). Other widths lost a microsecond in fifty to the turn.
  const int turn = (K & 2047) == 0 ? (int)(blockIdx.x >> 3) % chunks : 0;
  int load_at = (first_chunk + turn) % chunks;   // the chunk of the weight's rows that the next request reads
  unsigned pair_off = 0;                         // bytes from the wave's first pair to the pair of the next request
  int load_c = first_chunk, load_p = first_pair;
  const bool past_end = lr >= last_rows;         // in the run's last pair this lane's row belongs to the next run
  constexpr int KSTEPS = RES_CHUNK / 32;
  bf16x8 w[SETS][2][KSTEPS];
  auto load_next = [&](bf16x8 (&dst)[2][KSTEPS]) {
    // an offset past the view's end reads zero and fetches nothing
    const bool dead = past_end && load_p == run_pairs - 1;
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
#pragma unroll
      for (int i = 0; i < KSTEPS; ++i)
        dst[rt][i] = w_view.load(dead ? 0xFFFFFFF0u : w_off[rt] + pair_off + (unsigned)load_at * (RES_CHUNK * 2) + i * 64);
    if (++load_at == chunks) load_at = 0;
    if (++load_c == chunks) {
      load_c = 0;
      ++load_p;
      pair_off += 64u * (unsigned)K;
    }
  };

  {  // Activations: 16-byte pieces in row-major order, 256 a pass, BATCH passes requested together. The weights
     // of the first SETS - 1 units are requested right after the first batch: loads return in order, so the
     // copy into LDS waits for its own loads only and the weights stay on their way through the barrier.
    const BufferView a_view = buffer_view(A, ((unsigned long long)(M - 1) * lda + K) * 2);
    const int k8 = K / 8, pieces = M * k8;
    const int row_step = 256 / k8, col_step = 256 % k8;
    int row = tid / k8, col = tid % k8;
    constexpr int BATCH = 16;
    bf16x8 stage[BATCH];
    int at[BATCH];
    auto request = [&]() {
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        at[j] = row < M ? row * row_elems + col * 8 : -1;
        stage[j] = a_view.load((unsigned)((row * lda + col * 8) * 2));  // a row past the last reads zero
        row += row_step;
        col += col_step;
        if (col >= k8) {
          col -= k8;
          ++row;
        }
      }
    };
    auto copy = [&]() {
#pragma unroll
      for (int j = 0; j < BATCH; ++j)
        if (at[j] >= 0) *(bf16x8*)(acts + at[j]) = stage[j];
    };
    // the sums of squares are requested first of all and added after the other requests, so that adding them waits
    // for nothing else
    Squares squares;
    if constexpr (SCALED) squares = request_squares(sumsq, groups, tid);
    request();
    // unconditionally (a stretch shorter than the pipeline requests units past its end, which it does not use:
    // memory of the next pairs, or nothing past the weight's end): behind a branch these loads would make the
    // copy below wait for them, since the compiler could not tell how many are in flight
    static_for<SETS - 1>([&](auto j) { load_next(w[j.value]); });
    if constexpr (SCALED) add_squares(squares, groups, tid, norm_part);
    copy();
    for (int base = 256 * BATCH; base < pieces; base += 256 * BATCH) {
      request();
      copy();
    }
  }
  __syncthreads();

  // a token past M gives a column of the instruction that is never stored: its lanes read the last row
  const int token = min(lr, M - 1);
  float inv = 1.f;
  if constexpr (SCALED) inv = inv_rms(norm_part, token, K, eps);
  const __bf16* a_lane = acts + token * row_elems + lg * 8;
  f32x4 acc[2] = {f32x4{0.f, 0.f, 0.f, 0.f}, f32x4{0.f, 0.f, 0.f, 0.f}};
  int mul_c = first_chunk, mul_p = first_pair;
  int mul_at = (first_chunk + turn) % chunks;   // the chunk of the activations that goes with the next unit
  bool first_part = true, from_start = first_chunk == 0;
  auto flush = [&](bool to_end) {  // the sums of units [from_start ? 0 : first_chunk, mul_c) of pair mul_p
    if (from_start && to_end) {
      store_gated(C, ldc, lr, o_begin + mul_p * 16 + lg * 4, M, o_end, acc[0] * inv, acc[1] * inv);
    } else {
      f32x4* dst = partial + (wave * 2 + (first_part ? 0 : 1)) * 2 * 64;
      dst[lane] = acc[0];
      dst[64 + lane] = acc[1];
    }
    acc[0] = acc[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    first_part = false;
    from_start = true;
    mul_c = 0;
    ++mul_p;
  };
  auto multiply = [&](const bf16x8 (&wf)[2][KSTEPS]) {
    const __bf16* a = a_lane + mul_at * RES_CHUNK;
#pragma unroll
    for (int i = 0; i < KSTEPS; ++i) {
      const bf16x8 av = *(const bf16x8*)(a + i * 32);
      acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[0][i], av, acc[0], 0, 0, 0);
      acc[1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[1][i], av, acc[1], 0, 0, 0);
    }
    ++mul_c;
    if (++mul_at == chunks) mul_at = 0;
  };
  auto step = [&](auto set_, auto rem_, int) {
    constexpr int SET = decltype(set_)::value, REM = decltype(rem_)::value;
    if constexpr (REM >= SETS - 1) load_next(w[(SET + SETS - 1) % SETS]);
    multiply(w[SET]);
    if constexpr (REM == 0) {
      flush(mul_c == chunks);
    } else {
      if (mul_c == chunks) flush(true);
    }
  };
  if (count >= SETS - 1) {
    run_pipeline<SETS, SETS - 1>(step, count);
  } else {  // fewer units than the pipeline is deep: all of them were requested above
    static_for<SETS - 1>([&](auto j) {
      if (j.value < count) {
        multiply(w[j.value]);
        if (j.value == count - 1 || mul_c == chunks) flush(mul_c == chunks);
      }
    });
  }
  __syncthreads();
  // A pair that a stretch boundary cuts is finished by the wave that holds its first unit: its own part,
  // then the first parts of the waves that follow, while they begin inside the pair.
  if (wave < 3 && u1 % chunks != 0) {
    const int p = u1 / chunks;
    if (p * chunks >= u0 && count > 0) {
      const f32x4* mine = partial + (wave * 2 + (p == first_pair ? 0 : 1)) * 2 * 64;
      f32x4 gate = mine[lane], up = mine[64 + lane];
      for (int w2 = wave + 1; w2 < 4 && bound(w2) < (p + 1) * chunks; ++w2) {
        if (bound(w2 + 1) == bound(w2)) continue;
        const f32x4* theirs = partial + w2 * 2 * 2 * 64;
        gate += theirs[lane];
        up += theirs[64 + lane];
      }
      store_gated(C, ldc, lr, o_begin + p * 16 + lg * 4, M, o_end, gate * inv, up * inv);
    }
  }
}

// Whether the resident kernel takes the shape, and the LDS it asks for (0: it does not).
int resident_lds_bytes(int M, int N, int K) {
  if (M > 16 || (K % 128) || (N & 31)) return 0;
  const long long need = RES_HEAD_BYTES + (long long)M * (K + 8) * 2;
  if (need > 160 * 1024) return 0;
  return (int)(need > 82 * 1024 ? need : 82 * 1024);  // more than half a CU's LDS: one workgroup per CU
}

template <bool SCALED>
int launch_resident_gated(const __bf16* A, const __bf16* W, __bf16* C, int M, int N, int K, long long lda,
                          long long ldc, const float* sumsq, int norm_groups, float eps, hipStream_t s) {
  const int lds_bytes = resident_lds_bytes(M, N, K);
  if (!lds_bytes) return VK_UNSUPPORTED_SIZE;
  // chunks of 128 where 256 does not divide K, with one register set more: as many bytes on their way
  const bool halves = K % 256 != 0;
  auto kernel = halves ? gemm_resident_gated_kernel<VK_RESIDENT_SETS + 1, SCALED, 128>
                       : gemm_resident_gated_kernel<VK_RESIDENT_SETS, SCALED, 256>;
  static bool configured[2] = {false, false};
  if (!configured[halves]) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return (int)e;
    configured[halves] = true;
  }
  const int cus = compute_units();
  const int pairs = N / 32;
  const int groups = pairs < cus ? pairs : cus;
  // byte offsets from the first row that a wave needs are 32-bit: its run's pairs and one more, 64 rows each
  if (((long long)(pairs / groups) + 4) * 64 * K >= (1ll << 31)) return VK_UNSUPPORTED_SIZE;
  kernel<<<groups, 256, lds_bytes, s>>>(A, W, C, M, N, K, lda, ldc, sumsq, norm_groups, eps);
  VK_LAUNCH_CHECK();
  return 0;
}

// C (+)= sum over ranges of partial[range] (+ bias): ranges in ascending order, four columns per thread.
template <typename TC, bool ACCUMULATE>
__global__ void gemm_reduce_kernel(const float* __restrict__ partial, const float* __restrict__ bias,
                                   TC* __restrict__ C, int M, int N, long long ldc, int ranges, int vector_ok) {
  const int quads = (N + 3) / 4;
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)M * quads) return;
  const int m = (int)(idx / quads), n = (int)(idx % quads) * 4;
  f32x4 sum = {0.f, 0.f, 0.f, 0.f};
  const bool whole = n + 3 < N && (N & 3) == 0;
  if (whole) {
    // the first eight ranges are requested together (a clamped range is not added), the others one by one
    constexpr int AHEAD = 8;
    f32x4 ahead[AHEAD];
#pragma unroll
    for (int r = 0; r < AHEAD; ++r) ahead[r] = *(const f32x4*)(partial + ((size_t)min(r, ranges - 1) * M + m) * N + n);
#pragma unroll
    for (int r = 0; r < AHEAD; ++r)
      if (r < ranges) sum += ahead[r];
    for (int r = AHEAD; r < ranges; ++r) sum += *(const f32x4*)(partial + ((size_t)r * M + m) * N + n);
  } else {
    for (int r = 0; r < ranges; ++r) {
      const float* src = partial + ((size_t)r * M + m) * N + n;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < N) sum[j] += src[j];
    }
  }
  store4<TC, ACCUMULATE>(C, ldc, m, n, M, N, sum, bias, vector_ok != 0);
}

// The same sum for the residual (C float, += ) that also prepares the norm after it (see FollowNorm): grid
// (ceil(N / 1024), M), a workgroup adds the squares of its up to 1,024 columns of one token in a fixed tree and
// leaves them in sumsq[blockIdx.x][token].
__global__ __launch_bounds__(256) void gemm_reduce_follow_kernel(const float* __restrict__ partial,
                                                                 const float* __restrict__ bias, float* __restrict__ C,
                                                                 int M, int N, long long ldc, int ranges, int vector_ok,
                                                                 FollowNorm follow) {
  __shared__ float wave_sum[4];
  const int m = blockIdx.y, n = (blockIdx.x * 256 + threadIdx.x) * 4;
  float squares = 0.f;
  if (n < N) {
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};
    const bool whole = n + 3 < N && vector_ok;
    if (whole) {
      // Everything the thread reads is requested before anything is added: the first eight ranges' sums, the old
      // residual, the gain and the bias. The kernel is a few memory round trips long and little else, and a
      // load that waits behind an addition is one more of them.
      constexpr int AHEAD = 8;
      f32x4 ahead[AHEAD];
#pragma unroll
      for (int r = 0; r < AHEAD; ++r)
        ahead[r] = *(const f32x4*)(partial + ((size_t)min(r, ranges - 1) * M + m) * N + n);   // a clamped range is not added
      float* at = C + (size_t)m * ldc + n;
      const f32x4 old = *(const f32x4*)at;
      const f32x4 gain = *(const f32x4*)(follow.gain + n);
      const f32x4 b = bias ? *(const f32x4*)(bias + n) : f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < AHEAD; ++r)
        if (r < ranges) sum += ahead[r];
      for (int r = AHEAD; r < ranges; ++r) sum += *(const f32x4*)(partial + ((size_t)r * M + m) * N + n);
      f32x4 x;
      bf16x4 scaled;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        x[j] = sum[j] + b[j] + old[j];
        scaled[j] = (__bf16)(x[j] * gain[j]);
        squares += x[j] * x[j];
      }
      *(f32x4*)at = x;
      *(bf16x4*)(follow.scaled + (size_t)m * follow.ld_scaled + n) = scaled;
    } else {
      for (int r = 0; r < ranges; ++r) {
        const float* src = partial + ((size_t)r * M + m) * N + n;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (n + j < N) sum[j] += src[j];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (n + j < N) {
          float* at = C + (size_t)m * ldc + n + j;
          const float x = sum[j] + (bias ? bias[n + j] : 0.f) + *at;
          *at = x;
          follow.scaled[(size_t)m * follow.ld_scaled + n + j] = (__bf16)(x * follow.gain[n + j]);
          squares += x * x;
        }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) squares += __shfl_xor(squares, off);
  if ((threadIdx.x & 63) == 0) wave_sum[threadIdx.x >> 6] = squares;
  __syncthreads();
  if (threadIdx.x == 0)
    follow.sumsq[(size_t)blockIdx.x * follow.sumsq_stride + m] = wave_sum[0] + wave_sum[1] + wave_sum[2] + wave_sum[3];
}

// The sum of a split q/k/v product's K ranges with what gemm_qkv_rope_kernel does in its epilogue: (division by
// the root mean square of the norm before, if `sumsq`,) bias, rounding to bfloat16, rotation, cache write. Grid
// (ceil(units / 256), M): a thread owns four consecutive dims below half the width of a q or k head together with
// their partners, or four dims of a v head. Without `sumsq` bit for bit what gemm_reduce_kernel followed by
// rope_kvwrite_kernel leaves. Needs a head width that is a multiple of 8 and N a multiple of 4.
struct ReduceRope {
  QkvRope r;
  int sumsq_stride;
};
__global__ __launch_bounds__(256) void gemm_reduce_rope_kernel(const float* __restrict__ partial,
                                                               const float* __restrict__ bias, __bf16* __restrict__ C,
                                                               int M, int N, int K, long long ldc, int ranges,
                                                               ReduceRope rr) {
  const QkvRope& r = rr.r;
  const int hd = r.hd, half = hd / 2, quads = half / 4;
  const int rotated_units = (r.heads + r.kv_heads) * quads, units = rotated_units + r.kv_heads * (hd / 4);
  const int u = blockIdx.x * 256 + threadIdx.x, m = blockIdx.y;
  if (u >= units) return;
  const bool rotated = u < rotated_units;
  const int head = rotated ? u / quads : r.heads + r.kv_heads + (u - rotated_units) / (hd / 4);
  const int d0 = rotated ? (u % quads) * 4 : ((u - rotated_units) % (hd / 4)) * 4;
  const int lo_col = head * hd + d0, hi_col = lo_col + half;
  f32x4 lo = {0.f, 0.f, 0.f, 0.f}, hi = {0.f, 0.f, 0.f, 0.f};
  {
    // the first four ranges of both halves are requested together (a clamped range is not added; a v head reads
    // its own columns twice), the others one by one
    constexpr int AHEAD = 4;
    f32x4 ahead_lo[AHEAD], ahead_hi[AHEAD];
    const int hi_at = rotated ? hi_col : lo_col;
#pragma unroll
    for (int range = 0; range < AHEAD; ++range) {
      const float* src = partial + ((size_t)min(range, ranges - 1) * M + m) * N;
      ahead_lo[range] = *(const f32x4*)(src + lo_col);
      ahead_hi[range] = *(const f32x4*)(src + hi_at);
    }
#pragma unroll
    for (int range = 0; range < AHEAD; ++range)
      if (range < ranges) {
        lo += ahead_lo[range];
        hi += ahead_hi[range];
      }
    for (int range = AHEAD; range < ranges; ++range) {
      const float* src = partial + ((size_t)range * M + m) * N;
      lo += *(const f32x4*)(src + lo_col);
      hi += *(const f32x4*)(src + hi_at);
    }
  }
  if (r.sumsq) {
    float squares = 0.f;
    for (int g = 0; g < r.groups; ++g) squares += r.sumsq[(size_t)g * rr.sumsq_stride + m];
    const float inv = 1.0f / sqrtf(squares / (float)K + r.eps);
    lo *= inv;
    hi *= inv;
  }
  if (bias) {
    lo += *(const f32x4*)(bias + lo_col);
    if (rotated) hi += *(const f32x4*)(bias + hi_col);
  }
  const int pos = r.positions[m];
  int page = -1;
  if (r.k_cache && head >= r.heads) page = r.block_table[(size_t)r.entry_of_token[m] * r.table_width + pos / r.block_size];
  const int slot = pos % r.block_size;
  bf16x4 a, b;
  if (rotated) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float sn, cs;
      sincosf((float)pos * r.inv_freq[d0 + j], &sn, &cs);
      const float l = (float)(__bf16)lo[j], h = (float)(__bf16)hi[j];
      a[j] = (__bf16)(l * cs - h * sn);
      b[j] = (__bf16)(l * sn + h * cs);
    }
    *(bf16x4*)(C + (size_t)m * ldc + lo_col) = a;
    *(bf16x4*)(C + (size_t)m * ldc + hi_col) = b;
    if (page >= 0) {
      __bf16* at = r.k_cache + (((size_t)page * r.kv_heads + (head - r.heads)) * r.block_size + slot) * hd + d0;
      *(bf16x4*)at = a;
      *(bf16x4*)(at + half) = b;
    }
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) a[j] = (__bf16)lo[j];
    *(bf16x4*)(C + (size_t)m * ldc + lo_col) = a;
    if (page >= 0) {
      __bf16* at = r.v_cache + (((size_t)page * r.kv_heads + (head - r.heads - r.kv_heads)) * hd + d0) * r.block_size + slot;
#pragma unroll
      for (int j = 0; j < 4; ++j) at[(size_t)j * r.block_size] = a[j];
    }
  }
}

// The kernel that adds the `used` K ranges of a split product of up to 64 tokens: the plain sum, or the sum that also
// prepares the norm after the residual (`follow`), or the one that rotates q and k and writes the cache (`rope`).
template <typename TC, bool ACC>
int reduce_ranges(const float* partial, const float* bias, TC* C, int M, int N, int K, long long ldc, int used,
                  int vector_ok, hipStream_t s, const FollowNorm* follow, const ReduceRope* rope) {
  if constexpr (ACC && sizeof(TC) == 4) {
    if (follow) {
      gemm_reduce_follow_kernel<<<dim3((N + 1023) / 1024, M), 256, 0, s>>>(partial, bias, (float*)C, M, N, ldc, used,
                                                                           (N & 3) == 0 ? 1 : 0, *follow);
      VK_LAUNCH_CHECK();
      return 0;
    }
  }
  if constexpr (!ACC && sizeof(TC) == 2) {
    if (rope) {
      const int units = (rope->r.heads + rope->r.kv_heads) * (rope->r.hd / 8) + rope->r.kv_heads * (rope->r.hd / 4);
      gemm_reduce_rope_kernel<<<dim3((units + 255) / 256, M), 256, 0, s>>>(partial, bias, (__bf16*)C, M, N, K, ldc, used, *rope);
      VK_LAUNCH_CHECK();
      return 0;
    }
  }
  const long long threads = (long long)M * ((N + 3) / 4);
  gemm_reduce_kernel<TC, ACC><<<(int)((threads + 255) / 256), 256, 0, s>>>(partial, bias, C, M, N, ldc, used, vector_ok);
  VK_LAUNCH_CHECK();
  return 0;
}

template <int CB, int RT, typename TC, bool ACC>
int launch_mid_as(const __bf16* A, const __bf16* W, const float* bias, TC* C, float* partial, long long partial_floats,
                  int ranges, int forced_rows, int M, int N, int K, long long lda, long long ldc, int vector_ok,
                  hipStream_t s, const FollowNorm* follow = nullptr, const ReduceRope* rope = nullptr) {
  constexpr int CHUNK = mid_chunk(CB);
  constexpr int lds_bytes = 2 * CB * 16 * (CHUNK + 8) * (int)sizeof(__bf16);
  const int rows = RT == 2 ? 32 : forced_rows ? forced_rows : balanced_rows(M, N, 4, ranges < 1 ? 1 : ranges);  // per wave
  const int blocks = (N + 4 * rows - 1) / (4 * rows);
  if (ranges <= 1) {
    auto kernel = gemm_mid_kernel<CB, RT, TC, ACC>;
    static bool configured = false;
    if (!configured) {
      hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) return (int)e;
      configured = true;
    }
    kernel<<<dim3(blocks, 1), 256, lds_bytes, s>>>(A, W, bias, C, M, N, K, lda, ldc, K, 0, vector_ok, rows);
    VK_LAUNCH_CHECK();
    return 0;
  }
  if (!partial || (long long)ranges * M * N > partial_floats) return VK_UNSUPPORTED_SIZE;
  auto kernel = gemm_mid_kernel<CB, RT, float, false>;
  static bool configured_partial = false;
  if (!configured_partial) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return (int)e;
    configured_partial = true;
  }
  const int k_per_range = ((K + ranges - 1) / ranges + CHUNK - 1) / CHUNK * CHUNK;
  const int used = (K + k_per_range - 1) / k_per_range;
  kernel<<<dim3(blocks, used), 256, lds_bytes, s>>>(A, W, nullptr, partial, M, N, K, lda, N, k_per_range,
                                                    (long long)M * N, (N & 3) == 0 ? 1 : 0, rows);
  VK_LAUNCH_CHECK();
  return reduce_ranges<TC, ACC>(partial, bias, C, M, N, K, ldc, used, vector_ok, s, follow, rope);
}

template <typename TC, bool ACC>
int launch_mid(const __bf16* A, const __bf16* W, const float* bias, TC* C, float* partial, long long partial_floats,
               int ranges, int rows_per_wave, int M, int N, int K, long long lda, long long ldc, int vector_ok,
               hipStream_t s, const FollowNorm* follow = nullptr, const ReduceRope* rope = nullptr) {
  const int cb = (M + 15) / 16;
  // 108 to 116: one tile per wave with a forced number of rows (8 to 16), for tests and measurements
  const int forced = rows_per_wave >= 108 && rows_per_wave <= 116 ? rows_per_wave - 100 : 0;
#define VK_MID(CBV, RTV) return launch_mid_as<CBV, RTV, TC, ACC>(A, W, bias, C, partial, partial_floats, ranges, forced, M, N, K, lda, ldc, vector_ok, s, follow, rope)
  if (cb > 4 && (follow || rope)) return VK_UNSUPPORTED_SIZE;  // the kernels that add their ranges take 64 tokens
  if (rows_per_wave == 2) {
    switch (cb) { case 1: VK_MID(1, 2); case 2: VK_MID(2, 2); case 3: VK_MID(3, 2); case 4: VK_MID(4, 2);
                  case 5: VK_MID(5, 2); case 6: VK_MID(6, 2); case 7: VK_MID(7, 2); case 8: VK_MID(8, 2); }
  } else {
    switch (cb) { case 1: VK_MID(1, 1); case 2: VK_MID(2, 1); case 3: VK_MID(3, 1); case 4: VK_MID(4, 1);
                  case 5: VK_MID(5, 1); case 6: VK_MID(6, 1); case 7: VK_MID(7, 1); case 8: VK_MID(8, 1); }
  }
#undef VK_MID
  return VK_UNSUPPORTED_SIZE;
}

int g_tile_group_m = 0;   // 0: chosen by shape; else the rows of tiles per block of tile_of, for measurements

template <bool DIRECT, int BM, int BN, int WM, int WN, typename TC, bool ACC, bool GATED, int STAGES>
constexpr auto tile_kernel() {
  if constexpr (DIRECT) return gemm_tile_direct_kernel<BM, BN, WM, WN, TC, ACC, GATED, STAGES>;
  else return gemm_tile_kernel<BM, BN, WM, WN, TC, ACC, GATED>;
}

// DIRECT: the kernel that loads straight into LDS; K must be a multiple of 64. STAGES: its LDS stages.
template <int BM, int BN, int WM, int WN, typename TC, bool ACC, bool GATED, bool DIRECT = false, int STAGES = 2>
int launch_tile_as(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                   long long ldc, int vector_ok, int ranges, float* partial, hipStream_t s, const TileNorm& norm) {
  static_assert(DIRECT || STAGES == 2, "only the direct kernel has a third stage");
  constexpr int lds_bytes = DIRECT ? STAGES * (BM + BN) * DIRECT_ROW : 2 * (BM + BN) * ROW * (int)sizeof(__bf16);
  static_assert(lds_bytes + WM * WN * 64 * 4 <= 160 * 1024, "a CU has 160 KB of LDS (the stages and the norm's sums)");
  const int tiles_m = (M + BM - 1) / BM, tiles_n = (N + BN - 1) / BN;
  const long long total = (long long)tiles_m * tiles_n;
  const long long grid = (total + XCDS - 1) / XCDS * XCDS;
  if (grid > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  // the tiles that an XCD works on at one time: one per CU, or two where the stages' LDS lets two share a CU
  const long long at_once = (long long)(compute_units() / XCDS) * (lds_bytes * 2 <= 160 * 1024 ? 2 : 1);
  const int group_m = g_tile_group_m > 0 ? (g_tile_group_m < tiles_m ? g_tile_group_m : tiles_m)
                                         : tile_group_rows(tiles_m, grid / XCDS < at_once ? grid / XCDS : at_once, BM, BN);
  if (ranges <= 1 || GATED) {
    static bool configured = false;
    auto kernel = tile_kernel<DIRECT, BM, BN, WM, WN, TC, ACC, GATED, STAGES>();
    if (!configured) {
      hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) return (int)e;
      configured = true;
    }
    kernel<<<(int)grid, WM * WN * 64, lds_bytes, s>>>(A, W, bias, C, M, N, K, lda, ldc, tiles_m, tiles_n, group_m,
                                                      vector_ok, K, 0, norm);
    VK_LAUNCH_CHECK();
    return 0;
  }
  // K split over workgroups: float partial sums [range, M, N], then the ranges are added in ascending order
  if constexpr (!GATED) {
    static bool configured_partial = false;
    auto kernel = tile_kernel<DIRECT, BM, BN, WM, WN, float, false, false, STAGES>();
    if (!configured_partial) {
      hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
      if (e != hipSuccess) return (int)e;
      configured_partial = true;
    }
    const int k_per_range = ((K + ranges - 1) / ranges + BK - 1) / BK * BK;
    const int used = (K + k_per_range - 1) / k_per_range;
    kernel<<<dim3((unsigned)grid, used), WM * WN * 64, lds_bytes, s>>>(A, W, nullptr, partial, M, N, K, lda, N, tiles_m,
                                                                       tiles_n, group_m, (N & 3) == 0 ? 1 : 0,
                                                                       k_per_range, (long long)M * N, norm);
    VK_LAUNCH_CHECK();
    const long long threads = (long long)M * ((N + 3) / 4);
    gemm_reduce_kernel<TC, ACC><<<(int)((threads + 255) / 256), 256, 0, s>>>(partial, bias, C, M, N, ldc, used, vector_ok);
    VK_LAUNCH_CHECK();
  }
  return 0;
}

// Process-wide overrides for tests and measurements (vk_gemm_bf16_tile_config sets them): plain globals, read by
// every launch of the tiled kernel from any thread and not synchronised. Nothing on the serving path sets them; a
// program that does must not launch products from another thread meanwhile.
int g_tile_config = -1;  // -1: chosen by shape; else a tiling (see launch_tile) and g_tile_ranges force a plan, for measurements
int g_tile_ranges = 1;
int g_tile_stages = 0;   // 0: chosen by shape; 2 or 3 force the direct kernel's LDS stages where the tiling has both

// Which tiling, and into how many ranges K is split: the pair with the shortest estimated time. A full GPU
// of 256x256 tiles runs at about 1.15 PFLOP/s with the kernel that loads straight into LDS and at 1.0
// with the staged one (measured on the 7B shapes at 2,048 tokens); the smaller tiles reach 0.75 to 0.8 of
// their kernel's best, 256x192 about 0.9, and 256x128 with its three LDS stages about 0.95 (it is what the output
// and down projections of 512 to 2,048 tokens run on, where 256x256 tiles are too few). Workgroups run in whole rounds of one per CU (two where
// the LDS of the tile's stages lets two share a CU: the 128x128 tile and its narrower kin with two stages, unless every workgroup finds a CU of its own), so a launch that fills
// the last round badly loses that share. Splitting K
// multiplies the workgroups, at the price of writing and re-reading float partial sums (they mostly stay
// in the caches: about 6 TB/s) and one more launch; each range keeps at least 512 of K. The estimate ranks
// the plans as measurements at 128 to 2,048 tokens do. Few tokens keep the token side of the tile at 128.
// Ties go to the larger tile and to fewer ranges.
// Past 128 tokens the estimate is fitted to a sweep of every tiling and split over the q/k/v, output, down and
// gate/up products of the seven Qwen2.5 shapes at 160 to 4,096 tokens (the plans it picks cost 1 % more time than
// the fastest ones together, 15 % at worst; with a share of time lost in proportion to the unfilled share it was
// 4 and 47 %): the work is that of whole tiles; a launch that fills its rounds to a share f runs at f^0.6 of the
// full rate, not f, because the CUs that are at work run faster when others are idle (what is limited is the
// chip, not the CU); a workgroup alone on a CU that could hold two runs at 0.75 of its share; the 128x128 tile on
// eight waves is worth 0.95, 256x128 1.05 and 256x192 1.1; a range of a split costs three passes over the output.
struct TilePlan { int config, ranges; };
int g_compute_units = 0;
// the 128-token tiles of the direct kernel run with a third LDS stage for up to 128 tokens (see launch_tile)
bool tile_is_deep(int M) { return g_tile_stages ? g_tile_stages == 3 : M <= 128; }
TilePlan choose_tile_plan(int M, int N, int K, long long partial_floats, bool direct, bool gated = false) {
  if (g_compute_units == 0) {
    int device = 0, count = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count <= 0)
      count = 256;
    g_compute_units = count;
  }
  struct Tiling { int config, tokens, rows; double speed; };
  static const Tiling staged[] = {{4, 256, 256, 1.0}, {2, 256, 128, 0.8}, {3, 128, 256, 0.8}, {0, 128, 128, 0.75}};
  // the last three (the gated product of up to 128 tokens only): the weight of a feed-forward has so many rows
  // that with 128 of them a tile the tiles come in more than one round and less than two (7B width at 64 tokens:
  // 296 tiles of 128 rows, two to a CU on 40 CUs, one on the others); a width of 96, 160 or 224 rows can come
  // close to one tile per CU (237 tiles of 160 rows)
  static const Tiling straight[] = {{5, 256, 256, 1.15}, {7, 256, 128, 1.1}, {8, 128, 256, 0.88}, {9, 128, 128, 0.9},
                                    {6, 256, 192, 1.05}, {10, 128, 96, 0.85}, {11, 128, 160, 0.88}, {12, 128, 224, 0.88}};
  const Tiling* tilings = direct ? straight : staged;
  TilePlan best{tilings[3].config, 1};
  double best_time = 1e30;
  const double flops = 2.0 * M * N * (double)K, output_bytes = 4.0 * M * N;
  const bool many = M > 128 && direct;   // the fitted estimate
  // Up to 128 tokens the plain product is a stream of the weights, and its estimate counts bytes: the weight rows
  // of whole tiles once, the activations once per tile of rows at half price (they come from L2), at 5.5 TB/s
  // times f^0.5 for rounds filled to a share f, the 128x256 tile a tenth faster than 128x128 (the 32B down
  // projection at 65 tokens: 128x256 in eight ranges 64.8 us, 128x128 in four, which the estimate by arithmetic
  // picked, 78.8; a sweep of both tiles and all splits over the products of the seven Qwen2.5 shapes at 65, 96
  // and 128 tokens: the plan picked is 3 % off the fastest at worst, 41 % before).
  const bool few = M <= 128 && direct && !gated;
  for (int i = 0; i < (direct ? (gated && M <= 128 ? 8 : 5) : 4); ++i) {
    const Tiling& t = tilings[i];
    if (M <= 128 && t.tokens > 128) continue;
    if (M > 128 && t.tokens == 128 && t.rows == 256) continue;  // with many tokens the wide side goes to the tokens
    const long long groups = (long long)((M + t.tokens - 1) / t.tokens) * ((N + t.rows - 1) / t.rows);
    // how many workgroups share a CU follows from the LDS of the stages that will be launched (at most two)
    const int stages = !direct ? 2 : t.tokens == 128 ? (tile_is_deep(M) ? 3 : 2) : (t.config == 7 && g_tile_stages != 2 ? 3 : 2);
    const int lds_bytes = stages * (t.tokens + t.rows) * (direct ? 128 : 144);
    const int resident = lds_bytes * 2 <= 160 * 1024 ? 2 : 1;
    for (int ranges = 1; ranges <= 8; ranges *= 2) {
      if (ranges > 1 && (K / ranges < 512 || (long long)ranges * M * N > partial_floats)) break;
      // workgroups that all find a CU of their own do not share one, however many would fit
      const long long slots = groups * ranges <= g_compute_units ? g_compute_units : (long long)g_compute_units * resident;
      const long long rounds = (groups * ranges + slots - 1) / slots;
      const double fill = (double)(groups * ranges) / ((double)rounds * slots);
      double time;
      if (many) {
        double speed = t.config == 9 ? 0.95 : t.config == 6 ? 1.1 : t.config == 7 ? 1.05 : t.speed;
        if (resident == 2 && groups * ranges <= g_compute_units) speed *= 0.75;
        // the work of whole tiles: rows past M or N are multiplied like the others
        const double tile_flops = 2.0 * (double)groups * t.tokens * t.rows * (double)K;
        time = tile_flops / (1e15 * speed * pow(fill, 0.6));
        if (ranges > 1) time += (3.0 * ranges + 1.0) * output_bytes / 6e12;
      } else if (few) {
        const double row_tiles = (double)((N + t.rows - 1) / t.rows);
        const double bytes = row_tiles * t.rows * (double)K * 2.0 + 0.5 * row_tiles * M * (double)K * 2.0;
        time = bytes / (5.5e12 * (t.config == 8 ? 1.1 : 1.0) * sqrt(fill));
        if (ranges > 1) time += (3.0 * ranges + 1.0) * output_bytes / 6e12;
      } else {
        time = flops / (1e15 * t.speed * fill);
        if (ranges > 1) time += (2.0 * ranges + 1.0) * output_bytes / 6e12 + 4e-6;
      }
      if (time < best_time * (1.0 - 1e-9)) {
        best_time = time;
        best = TilePlan{t.config, ranges};
      }
    }
  }
  return best;
}

// Tilings: 0, 2, 3, 4 the staged kernel at 128x128, 256x128, 128x256, 256x256; 9, 7, 8, 5 the same tiles
// with the kernel that loads straight into LDS, which needs K to be a multiple of 64, and 6 that kernel at
// 256x192 (2,048 tokens x 4,608 rows are 192 such tiles for 256 CUs, against 144 of 256x256).
template <typename TC, bool ACC, bool GATED = false>
int launch_tile(const __bf16* A, const __bf16* W, const float* bias, TC* C, int M, int N, int K, long long lda,
                long long ldc, int vector_ok, float* partial, long long partial_floats, hipStream_t s,
                const TileNorm& norm = TileNorm{}) {
  const bool direct = (K & 63) == 0;
  TilePlan plan = choose_tile_plan(M, N, K, (GATED || !partial) ? 0 : partial_floats, direct, GATED);
  if (g_tile_config >= 0) plan = TilePlan{g_tile_config, g_tile_ranges > 1 && !GATED && partial ? g_tile_ranges : 1};
  if (plan.ranges > 1 && (long long)plan.ranges * M * N > partial_floats) plan.ranges = 1;
  if (plan.config >= 10 && !GATED) plan.config = 9;   // the narrow tiles exist for the gated product only
  if (!direct) {
    switch (plan.config) { case 5: case 6: plan.config = 4; break; case 7: plan.config = 2; break; case 8: plan.config = 3; break;
                           case 9: case 10: case 11: case 12: plan.config = 0; break; }
  }
  const int r = plan.ranges;
#define VK_TILE(BMV, BNV, WMV, WNV, DIRECTV) \
  return launch_tile_as<BMV, BNV, WMV, WNV, TC, ACC, GATED, DIRECTV>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, r, partial, s, \
                                                                     norm)
  // the 128-token tiles of the direct kernel with a third LDS stage: up to 128 tokens the product is a stream of
  // the weights (with more tokens, and so more tiles per weight row, two stages measured the same or better)
#define VK_TILE_DEEP(BMV, BNV, WMV, WNV)                                                                              \
  {                                                                                                                  \
    if (deep)                                                                                                        \
      return launch_tile_as<BMV, BNV, WMV, WNV, TC, ACC, GATED, true, 3>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, r, \
                                                                         partial, s, norm);                          \
    VK_TILE(BMV, BNV, WMV, WNV, true);                                                                               \
  }
  const bool deep = tile_is_deep(M);
  if constexpr (GATED) {
    switch (plan.config) {
      // four waves side by side along the tokens: a wave owns all rows of the tile, an even number of 16-row
      // tiles, so gate and up rows of the same outputs meet in one wave
      case 10: VK_TILE_DEEP(128, 96, 4, 1);
      case 11: VK_TILE_DEEP(128, 160, 4, 1);
      case 12: VK_TILE_DEEP(128, 224, 4, 1);
    }
  }
  switch (plan.config) {
    case 5: VK_TILE(256, 256, 4, 2, true);
    case 6: VK_TILE(256, 192, 4, 2, true);
    case 7:  // three stages fit this tile's LDS, and its loads per product are the most of the 256-token tiles
      if (g_tile_stages != 2)
        return launch_tile_as<256, 128, 4, 2, TC, ACC, GATED, true, 3>(A, W, bias, C, M, N, K, lda, ldc, vector_ok, r,
                                                                       partial, s, norm);
      VK_TILE(256, 128, 4, 2, true);
    case 8: VK_TILE_DEEP(128, 256, 2, 4);
    case 9:
      // past 128 tokens eight waves of 32 x 64 instead of four of 64 x 64: such tiles run where the tiles are few, often
      // one workgroup to a CU, and twice the waves hide more of its waits (2,048 tokens on 2,048 x 2,048: 30.1 to
      // 26.9 us, 512 tokens on 2,048 x 1,536: 16.5 to 12.1; nowhere slower)
      if (!deep) VK_TILE(128, 128, 4, 2, true);
      VK_TILE_DEEP(128, 128, 2, 2);
    case 2: VK_TILE(256, 128, 4, 2, false);
    case 3: VK_TILE(128, 256, 2, 4, false);
    case 4: VK_TILE(256, 256, 4, 4, false);
    default: VK_TILE(128, 128, 2, 2, false);
  }
#undef VK_TILE_DEEP
#undef VK_TILE
}
}  // namespace

// A, W: bfloat16. c_dtype: 0 float, 1 bfloat16. accumulate needs a float C. Requirements (checked here):
// K a multiple of 8 and lda a multiple of 8 (16-byte chunks); A and W 16-byte aligned.
// `skinny_limit`: M at or below it takes the weight-streaming kernel (at most 64).
// `skinny_shape`: 0 lets the launcher choose the row tiles per wave and the rows per workgroup; 1 or 2 force one
// or two tiles; 108 to 116 force one tile and 8 to 16 rows per workgroup.
// `partial` (may be null): a float workspace of `partial_floats` floats that the tiled kernel may split K into.
extern "C" int vk_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N, int K,
                            long long lda, long long ldc, int accumulate, int skinny_limit, int skinny_shape,
                            float* partial, long long partial_floats, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 23) || lda >= (1 << 23)) return VK_UNSUPPORTED_SIZE;  // byte offsets inside a tile of 256 rows are 32-bit
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
                    : launch_tile<float, true>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, partial, partial_floats, s);
    return skinny ? launch_skinny<float, false>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, skinny_shape, s)
                  : launch_tile<float, false>(a, w, bias, (float*)C, M, N, K, lda, ldc, vector_ok, partial, partial_floats, s);
  }
  if (c_dtype == DT_BF16)
    return skinny ? launch_skinny<__bf16, false>(a, w, bias, (__bf16*)C, M, N, K, lda, ldc, vector_ok, skinny_shape, s)
                  : launch_tile<__bf16, false>(a, w, bias, (__bf16*)C, M, N, K, lda, ldc, vector_ok, partial, partial_floats, s);
  return VK_BAD_ARGUMENT;
}

// The same product for M <= 128 with the activations shared through LDS. `ranges` > 1 splits K over
// workgroups: partial sums go to `partial` (at least ranges * M * N floats) and a second kernel adds them.
// rows_per_wave: 1 or 2 tiles of 16 weight rows per wave; with 1 the launcher may give a wave fewer than 16 rows
// (balanced_rows), and 108 to 116 force one tile with 8 to 16 rows.
static int gemm_mid_checked(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N, int K,
                            long long lda, long long ldc, int accumulate, int ranges, int rows_per_wave,
                            float* partial, long long partial_floats, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 128) return VK_UNSUPPORTED_SIZE;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N || ranges < 1) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || ((uintptr_t)partial & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 24) || lda >= (1 << 24)) return VK_UNSUPPORTED_SIZE;  // byte offsets inside a tile of rows are 32-bit
  if (accumulate && c_dtype != DT_F32) return VK_BAD_ARGUMENT;
  const int elem = c_dtype == DT_F32 ? 4 : 2;
  const int vector_ok = ((ldc & 3) == 0 && ((uintptr_t)C & (4 * elem - 1)) == 0 &&
                         (bias == nullptr || ((uintptr_t)bias & 15) == 0)) ? 1 : 0;
  hipStream_t s = (hipStream_t)stream;
  const __bf16* a = (const __bf16*)A;
  const __bf16* w = (const __bf16*)W;
  if (c_dtype == DT_F32) {
    if (accumulate)
      return launch_mid<float, true>(a, w, bias, (float*)C, partial, partial_floats, ranges, rows_per_wave, M, N, K, lda, ldc, vector_ok, s);
    return launch_mid<float, false>(a, w, bias, (float*)C, partial, partial_floats, ranges, rows_per_wave, M, N, K, lda, ldc, vector_ok, s);
  }
  if (c_dtype == DT_BF16)
    return launch_mid<__bf16, false>(a, w, bias, (__bf16*)C, partial, partial_floats, ranges, rows_per_wave, M, N, K, lda, ldc, vector_ok, s);
  return VK_BAD_ARGUMENT;
}

extern "C" int vk_gemm_bf16_mid(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N,
                                int K, long long lda, long long ldc, int accumulate, int ranges, int rows_per_wave,
                                float* partial, long long partial_floats, void* stream) {
  return gemm_mid_checked(A, W, bias, C, c_dtype, M, N, K, lda, ldc, accumulate, ranges, rows_per_wave, partial,
                          partial_floats, stream);
}

// --- the split-K product without a workspace argument (declared in no_alloc.h) ---------------------------------
// The partial sums of the K ranges live in this array, which every GPU that loads the library holds at an
// address of its own until the process ends. In host code the array's name stands for the symbol, not for device
// memory: its address on the current device is asked for once per device and only that pointer is ever used.
static __device__ __align__(256) float scratch[VK_NO_ALLOC_SCRATCH_FLOATS];

namespace {
constexpr int NO_ALLOC_MAX_DEVICES = 64;
float* g_scratch_of_device[NO_ALLOC_MAX_DEVICES] = {};
std::mutex g_scratch_lock;

// The array's address on the current device; nullptr and `*status` set when it cannot be had.
float* scratch_of_current_device(int* status) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) { *status = (int)e; return nullptr; }
  if (device < 0 || device >= NO_ALLOC_MAX_DEVICES) { *status = VK_UNSUPPORTED_SIZE; return nullptr; }
  std::lock_guard<std::mutex> hold(g_scratch_lock);
  if (!g_scratch_of_device[device]) {
    float* address = nullptr;
    e = hipGetSymbolAddress((void**)&address, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !address) { *status = e != hipSuccess ? (int)e : VK_BAD_ARGUMENT; return nullptr; }
    g_scratch_of_device[device] = address;
  }
  return g_scratch_of_device[device];
}
}  // namespace

extern "C" long long vk_gemm_bf16_mid_no_alloc_capacity() { return VK_NO_ALLOC_SCRATCH_FLOATS; }

extern "C" int vk_gemm_bf16_mid_no_alloc(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M,
                                         int N, int K, long long lda, long long ldc, int accumulate, int ranges,
                                         int rows_per_wave, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (ranges < 1) return VK_BAD_ARGUMENT;
  if (M > 128) return VK_UNSUPPORTED_SIZE;   // as vk_gemm_bf16_mid; checked before M enters a product
  // every range writes all of its M x N sums before the second kernel reads them, so nothing has to be cleared;
  // each factor is bounded before the product is formed (M <= 128), so the comparison cannot overflow
  if (ranges > 1 && ((long long)ranges > VK_NO_ALLOC_SCRATCH_FLOATS || (long long)N > VK_NO_ALLOC_SCRATCH_FLOATS ||
                     (long long)ranges * M * N > VK_NO_ALLOC_SCRATCH_FLOATS))
    return VK_UNSUPPORTED_SIZE;
  int status = 0;
  float* partial = scratch_of_current_device(&status);
  if (!partial) return status;
  return gemm_mid_checked(A, W, bias, C, c_dtype, M, N, K, lda, ldc, accumulate, ranges, rows_per_wave, partial,
                          VK_NO_ALLOC_SCRATCH_FLOATS, stream);
}

// out[M, N / 2] = up * silu(gate) of the product with a fused gate/up weight W[N, K] whose rows are
// interleaved in groups of 16 (see store_gated). bfloat16 in and out; N a multiple of 32.
// More than 64 tokens: the tiled kernel; up to 64: the LDS-shared kernel with one K range and `rows_per_wave`
// (1 or 2) tiles of 16 rows per wave, or with `rows_per_wave` 0 the kernel that keeps the activations resident
// in LDS (up to 16 tokens, K a multiple of 128, tokens x K within LDS; anything else is refused), or with
// `rows_per_wave` 3 the tiled kernel.
extern "C" int vk_gemm_bf16_gated(const void* A, const void* W, void* C, int M, int N, int K, long long lda,
                                  long long ldc, int rows_per_wave, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || (N & 31) || ldc < N / 2) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 23) || lda >= (1 << 23)) return VK_UNSUPPORTED_SIZE;  // byte offsets inside a tile of 256 rows are 32-bit
  hipStream_t s = (hipStream_t)stream;
  const __bf16* a = (const __bf16*)A;
  const __bf16* w = (const __bf16*)W;
  __bf16* c = (__bf16*)C;
  if (M > 64 || rows_per_wave == 3) return launch_tile<__bf16, false, true>(a, w, nullptr, c, M, N, K, lda, ldc, 0, nullptr, 0, s);
  if (rows_per_wave == 0) return launch_resident_gated<false>(a, w, c, M, N, K, lda, ldc, nullptr, 0, 0.f, s);
  const int cb = (M + 15) / 16;
#define VK_GATED(CBV, RTV)                                                                                         \
  {                                                                                                                \
    constexpr int lds_bytes = 2 * CBV * 16 * MID_ROW * (int)sizeof(__bf16);                                       \
    auto kernel = gemm_mid_kernel<CBV, RTV, __bf16, false, true>;                                                  \
    static bool configured = false;                                                                                \
    if (!configured) {                                                                                             \
      hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes); \
      if (e != hipSuccess) return (int)e;                                                                          \
      configured = true;                                                                                           \
    }                                                                                                              \
    kernel<<<dim3((N + 64 * RTV - 1) / (64 * RTV), 1), 256, lds_bytes, s>>>(a, w, nullptr, c, M, N, K, lda, ldc, K, 0, 0, 16 * RTV); \
    VK_LAUNCH_CHECK();                                                                                             \
    return 0;                                                                                                      \
  }
  if (rows_per_wave == 2) {
    switch (cb) { case 1: VK_GATED(1, 2) case 2: VK_GATED(2, 2) case 3: VK_GATED(3, 2) case 4: VK_GATED(4, 2) }
  } else {
    switch (cb) { case 1: VK_GATED(1, 1) case 2: VK_GATED(2, 1) case 3: VK_GATED(3, 1) case 4: VK_GATED(4, 1) }
  }
#undef VK_GATED
  return VK_UNSUPPORTED_SIZE;
}

// qkv[M, N] = A W^T + bias in bfloat16 for up to 16 tokens, its q and k heads rotated (full rotation: inv_freq
// holds hd / 2 floats) and the tokens' K and V stored in their pages, as vk_gemm_bf16 followed by vk_rope_kvwrite
// would leave them. N = (heads + 2 kv_heads) hd, hd even. k_cache null: no cache is written.
// K pages [page, kv_head, slot, hd], V pages [page, kv_head, hd, slot]; a negative page id writes nothing.
// `sumsq` (may be null): A is x * gain of the norm before the product as vk_gemm_bf16_follow or
// vk_gemm_bf16_mid_follow left it, with `norm_groups` sums of squares; the sums of the product are divided by
// the root mean square (`eps` inside the root) before the bias.
extern "C" int vk_gemm_bf16_qkv_rope(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                                     long long lda, long long ldc, const int* positions, const float* inv_freq,
                                     void* k_cache, void* v_cache, const int* entry_of_token, const int* block_table,
                                     int table_width, int block_size, int heads, int kv_heads, int hd,
                                     const float* sumsq, int norm_groups, float eps, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (M > 16) return VK_UNSUPPORTED_SIZE;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (heads <= 0 || kv_heads <= 0 || hd <= 0 || (hd & 1) || (long long)(heads + 2 * kv_heads) * hd != N || !positions ||
      !inv_freq)
    return VK_BAD_ARGUMENT;
  if (k_cache && (!v_cache || !entry_of_token || !block_table || table_width <= 0 || block_size <= 0)) return VK_BAD_ARGUMENT;
  // byte offsets are 32-bit, and bit 31 switches a lane's row off
  if ((long long)N * K * 2 >= (1ll << 31) || lda >= (1 << 23)) return VK_UNSUPPORTED_SIZE;
  int pairs = 8, values = 16, groups = 1;
  qkv_rope_plan(M, heads, kv_heads, hd, &pairs, &values, &groups);
  if (sumsq && (norm_groups <= 0 || norm_groups > 512 || ((uintptr_t)sumsq & 15))) return VK_BAD_ARGUMENT;
  const QkvRope r{positions, inv_freq, (__bf16*)k_cache, (__bf16*)v_cache, entry_of_token, block_table,
                  table_width, block_size, heads, kv_heads, hd, pairs, values, sumsq, norm_groups, eps};
  const bool one_tile = values <= 2 * (8 - pairs);
#define VK_QKV(RTV, SCALEDV)                                                                                          \
  gemm_qkv_rope_kernel<RTV, SCALEDV><<<groups, 256, 0, (hipStream_t)stream>>>((const __bf16*)A, (const __bf16*)W, bias, \
                                                                              (__bf16*)C, M, N, K, lda, ldc, r)
  if (sumsq) {
    if (one_tile) VK_QKV(1, true); else VK_QKV(2, true);
  } else {
    if (one_tile) VK_QKV(1, false); else VK_QKV(2, false);
  }
#undef VK_QKV
  VK_LAUNCH_CHECK();
  return 0;
}

// C += A W^T + bias for up to 16 tokens (C float: the residual), and what the RMS norm after it needs (see
// FollowNorm): scaled[M, N] = bfloat16(C * gain) with row stride ld_scaled, and the workgroups' sums of squares,
// sumsq[*groups][16] floats (`sumsq_floats`: the room there is). *groups receives the number of workgroups.
extern "C" int vk_gemm_bf16_follow(const void* A, const void* W, const float* bias, float* C, int M, int N, int K,
                                   long long lda, long long ldc, const float* gain, void* scaled, long long ld_scaled,
                                   float* sumsq, long long sumsq_floats, int* groups, void* stream) {
  if (M <= 0 || N <= 0 || M > 16) return VK_UNSUPPORTED_SIZE;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N || ld_scaled < N || !gain || !scaled || !sumsq || !groups)
    return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 23) || lda >= (1 << 23)) return VK_UNSUPPORTED_SIZE;
  const int vector_ok = ((ldc & 3) == 0 && ((uintptr_t)C & 15) == 0 && (bias == nullptr || ((uintptr_t)bias & 15) == 0) &&
                         ((uintptr_t)gain & 15) == 0 && (ld_scaled & 3) == 0 && ((uintptr_t)scaled & 7) == 0) ? 1 : 0;
  int rows = balanced_rows(M, N, 1, 1);
  if ((N + rows - 1) / rows > 512) rows = 16;  // the product after the norm adds at most 512 groups
  const int blocks = (N + rows - 1) / rows;
  if (blocks > 512 || (long long)blocks * 16 > sumsq_floats) return VK_UNSUPPORTED_SIZE;
  *groups = blocks;
  gemm_skinny_kernel<1, 1, 4, float, true, VK_SKINNY_SETS, true><<<blocks, 256, 0, (hipStream_t)stream>>>(
      (const __bf16*)A, (const __bf16*)W, bias, C, M, N, K, lda, ldc, vector_ok, rows,
      FollowNorm{gain, (__bf16*)scaled, sumsq, ld_scaled});
  VK_LAUNCH_CHECK();
  return 0;
}

// vk_gemm_bf16_follow for up to 64 tokens where K is split over workgroups (vk_gemm_bf16_mid with `ranges` > 1
// into a float C with accumulation): the kernel that adds the ranges also leaves `scaled` and the sums of squares,
// here ceil(N / 1024) groups of `sumsq_stride` floats (16, or 64 for more than 16 tokens).
extern "C" int vk_gemm_bf16_mid_follow(const void* A, const void* W, const float* bias, float* C, int M, int N, int K,
                                       long long lda, long long ldc, int ranges, int rows_per_wave, float* partial,
                                       long long partial_floats, const float* gain, void* scaled, long long ld_scaled,
                                       float* sumsq, long long sumsq_floats, int sumsq_stride, int* groups, void* stream) {
  if (M <= 0 || N <= 0 || M > 64) return VK_UNSUPPORTED_SIZE;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N || ranges < 2 || ld_scaled < N || !gain || !scaled || !sumsq ||
      !groups || !partial)
    return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || ((uintptr_t)partial & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 24) || lda >= (1 << 24)) return VK_UNSUPPORTED_SIZE;
  if ((sumsq_stride != 16 && sumsq_stride != 64) || M > sumsq_stride) return VK_BAD_ARGUMENT;
  const int blocks = (N + 1023) / 1024;
  if ((long long)blocks * sumsq_stride > sumsq_floats) return VK_UNSUPPORTED_SIZE;
  // the ranges must really be split, or the product would write C without the kernel that adds them
  const int k_per_range = ((K + ranges - 1) / ranges + MID_CHUNK - 1) / MID_CHUNK * MID_CHUNK;
  if ((K + k_per_range - 1) / k_per_range < 2) return VK_UNSUPPORTED_SIZE;
  *groups = blocks;
  const FollowNorm follow{gain, (__bf16*)scaled, sumsq, ld_scaled, sumsq_stride};
  return launch_mid<float, true>((const __bf16*)A, (const __bf16*)W, bias, C, partial, partial_floats, ranges, rows_per_wave,
                                 M, N, K, lda, ldc, 0, (hipStream_t)stream, &follow);
}

// vk_gemm_bf16_qkv_rope for up to 64 tokens where K is split over workgroups (vk_gemm_bf16_mid with `ranges` > 1):
// the kernel that adds the ranges also divides by the norm's root mean square (if `sumsq`: `norm_groups` groups of
// `sumsq_stride` floats), adds the bias, rotates and writes the cache. hd a multiple of 8.
extern "C" int vk_gemm_bf16_mid_qkv_rope(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                                         long long lda, long long ldc, int ranges, int rows_per_wave, float* partial,
                                         long long partial_floats, const int* positions, const float* inv_freq,
                                         void* k_cache, void* v_cache, const int* entry_of_token, const int* block_table,
                                         int table_width, int block_size, int heads, int kv_heads, int hd,
                                         const float* sumsq, int norm_groups, int sumsq_stride, float eps, void* stream) {
  if (M <= 0 || N <= 0 || M > 64) return VK_UNSUPPORTED_SIZE;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || ldc < N || (ldc & 3) || ranges < 2 || !partial) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || ((uintptr_t)partial & 15) || ((uintptr_t)C & 7) ||
      ((uintptr_t)bias & 15) || ((uintptr_t)k_cache & 7))
    return VK_BAD_ARGUMENT;
  if (heads <= 0 || kv_heads <= 0 || hd <= 0 || (hd & 7) || (long long)(heads + 2 * kv_heads) * hd != N || !positions ||
      !inv_freq)
    return VK_BAD_ARGUMENT;
  if (k_cache && (!v_cache || !entry_of_token || !block_table || table_width <= 0 || block_size <= 0)) return VK_BAD_ARGUMENT;
  if (sumsq && (norm_groups <= 0 || (sumsq_stride != 16 && sumsq_stride != 64) || M > sumsq_stride)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 24) || lda >= (1 << 24)) return VK_UNSUPPORTED_SIZE;
  const int k_per_range = ((K + ranges - 1) / ranges + MID_CHUNK - 1) / MID_CHUNK * MID_CHUNK;
  if ((K + k_per_range - 1) / k_per_range < 2) return VK_UNSUPPORTED_SIZE;
  const ReduceRope rope{QkvRope{positions, inv_freq, (__bf16*)k_cache, (__bf16*)v_cache, entry_of_token, block_table,
                                table_width, block_size, heads, kv_heads, hd, 0, 0, sumsq, norm_groups, eps},
                        sumsq_stride};
  return launch_mid<__bf16, false>((const __bf16*)A, (const __bf16*)W, bias, (__bf16*)C, partial, partial_floats, ranges,
                                   rows_per_wave, M, N, K, lda, ldc, 0, (hipStream_t)stream, nullptr, &rope);
}

// vk_gemm_bf16_gated with resident activations (rows_per_wave 0) on the output of vk_gemm_bf16_follow: A = scaled,
// and gate and up are divided by the root mean square that `sumsq[groups][16]` and `eps` give before the activation.
extern "C" int vk_gemm_bf16_gated_scaled(const void* A, const void* W, void* C, int M, int N, int K, long long lda,
                                         long long ldc, const float* sumsq, int groups, float eps, void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || (N & 31) || ldc < N / 2 || !sumsq || groups <= 0) return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15) || ((uintptr_t)sumsq & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 23) || lda >= (1 << 23)) return VK_UNSUPPORTED_SIZE;
  if (groups > 512) return VK_UNSUPPORTED_SIZE;  // a thread adds two groups
  return launch_resident_gated<true>((const __bf16*)A, (const __bf16*)W, (__bf16*)C, M, N, K, lda, ldc, sumsq, groups, eps,
                                     (hipStream_t)stream);
}

// vk_gemm_bf16_gated on the tiled kernel for any number of tokens, with A = x * gain of the norm before and gate
// and up divided by the root mean square that `sumsq` (`groups` groups of `stride` floats) and `eps` give.
extern "C" int vk_gemm_bf16_gated_tile_scaled(const void* A, const void* W, void* C, int M, int N, int K, long long lda,
                                              long long ldc, const float* sumsq, int groups, int stride, float eps,
                                              void* stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || (K & 7) || (lda & 7) || lda < K || (N & 31) || ldc < N / 2 || !sumsq || groups <= 0 || stride < M)
    return VK_BAD_ARGUMENT;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return VK_BAD_ARGUMENT;
  if (K >= (1 << 23) || lda >= (1 << 23)) return VK_UNSUPPORTED_SIZE;
  TileNorm norm;
  norm.sumsq = sumsq;
  norm.groups = groups;
  norm.stride = stride;
  norm.eps = eps;
  return launch_tile<__bf16, false, true>((const __bf16*)A, (const __bf16*)W, nullptr, (__bf16*)C, M, N, K, lda, ldc, 0,
                                          nullptr, 0, (hipStream_t)stream, norm);
}

// For measurements: the rows of tiles per block of the tiled kernel's tile order (0: chosen by shape).
extern "C" int vk_gemm_bf16_tile_group(int rows) {
  if (rows < 0) return VK_BAD_ARGUMENT;
  g_tile_group_m = rows;
  return 0;
}

extern "C" int vk_gemm_bf16_tile_config(int tiling, int ranges, int stages) {
  if (stages != 0 && stages != 2 && stages != 3) return VK_BAD_ARGUMENT;
  g_tile_config = tiling;
  g_tile_ranges = ranges;
  g_tile_stages = stages;
  return 0;
}
