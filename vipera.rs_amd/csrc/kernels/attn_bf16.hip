// Causal grouped-query attention over the paged cache on the matrix cores (bfloat16 in, 32-bit
// scores, softmax and sums). Compiled once per padded head width: -DHDP=32..256 in steps of 32.
//
// What is computed is the reference's attention (crates/vipera-backend-cpu/src/model.rs:1811-1857):
// head h uses key head h / group; score = dot(q, k) * scale; a token at position p sees positions
// [lo, p], lo = 0 or p + 1 - window (model.rs:2509); output = softmax-weighted sum of V. The decode
// form splits the positions into chunks whose partial (max, sum, weighted sum) are merged afterwards,
// as the reference's split kernels do (crates/vipera-backend-gpu/src/layer.cu:307-467).
//
// A wave works on blocks of 16 columns and a range of positions. A column is a (token, query head)
// pair: 16 consecutive tokens of one head (prompts), or up to 16 query heads of one key head at one
// token (decoding; they share every K and V read). The decode kernel reads the cache straight into
// the instruction's operands; the prompt kernel shares K/V tiles among its waves through LDS. The operand layout
// of v_mfma_f32_16x16x32_bf16 (a lane holds 8 consecutive k of one row) is how K lies in the cache,
// [page, kv_head, slot, head_dim], and V is cached transposed, [page, kv_head, head_dim, slot], so
// that a lane reads consecutive positions of one output dim.
//     S^T = K Q^T : lane (c = l % 16, g = l / 16), register j  <->  S[row 4g + j of a 16-row tile][column c]
//     O^T = V^T P : the 32 positions of a step feed the instruction in the order the scores arrive in, and a
//                   sum does not care how its terms are numbered. Prompts: row r of tile t is position 16t + r
//                   (slot 8g + i <-> position 4g + i for i < 4, 16 + 4g + i - 4 for i >= 4), and the V^T tile
//                   is laid out in LDS in that order. Decoding: which position a K row holds is free, since every
//                   lane fetches its own row: row 4g + j of tile t is position 8g + 4t + j, so that a lane's eight
//                   weights are the eight consecutive positions 8g .. 8g + 7 and its V^T operand one 16-byte read.
// The softmax is online over steps of 32 positions that start at multiples of 32, so a token's
// arithmetic depends on its position and the cache only.
#include "common.h"
#include "pipeline.h"

#ifndef HDP
#define HDP 128
#endif

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

namespace {
// Until none of the wave's vector memory loads is in flight (s_waitcnt vmcnt(0), the other counters left alone).
// A barrier alone does not wait for loads that write LDS.
__device__ __forceinline__ void wait_own_loads() { __builtin_amdgcn_s_waitcnt(0x0F70); }

constexpr int KS = HDP / 32;  // instruction steps over the head width
constexpr int DT = HDP / 16;  // 16-wide tiles of the output width

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// A V^T operand with the elements of positions at or past a range's end set to zero: of its elements 0-3 the first
// `head` are kept, of its elements 4-7 the first `tail` (counts below 1 keep nothing, above 3 everything). Such a
// position's weight is zero, but the slot may hold anything, also what is not finite (a page that another request
// gave back, which the matrix instruction would turn into NaN: 0 * NaN), so the value is made zero as well. Only the
// last tile of a range needs it.
typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ bf16x8 keep_before_end(bf16x8 v, int head, int tail) {
  auto pair = [](int kept, int e) { return kept > e + 1 ? 0xFFFFFFFFu : kept > e ? 0x0000FFFFu : 0u; };
  const u32x4 mask = {pair(head, 0), pair(head, 2), pair(tail, 0), pair(tail, 2)};
  return __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, v) & mask);
}

// A column's four lanes (lanes c, c + 16, c + 32, c + 48) combine their values with two lane swaps that run in the
// vector ALU (v_permlane16_swap exchanges the odd 16-lane rows of one register with the even rows of another,
// v_permlane32_swap the upper half of one with the lower half of another; with both registers holding v, the two
// results hold a lane's own value and its partner's), not with two round trips through the LDS crossbar, which sat
// in the middle of every step's chain from scores to weights.
__device__ __forceinline__ float max_of_column(float v) {
  auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = fmaxf(__uint_as_float(rows[0]), __uint_as_float(rows[1]));
  auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(halves[0]), __uint_as_float(halves[1]));
}
// The sum in a fixed order: (lane group 0 + 1) + (2 + 3) for every lane.
__device__ __forceinline__ float sum_of_column(float v) {
  auto rows = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  v = __uint_as_float(rows[0]) + __uint_as_float(rows[1]);
  auto halves = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(halves[0]) + __uint_as_float(halves[1]);
}

// Position -> (page index, slot in the page). Page sizes are almost always powers of two: then a shift
// and a mask stand for the division, which would otherwise cost some thirty instructions per use, on
// the path to every load address.
struct PageSize {
  int size, shift;  // shift < 0: not a power of two
  __device__ __forceinline__ explicit PageSize(int block_size)
      : size(block_size), shift((block_size & (block_size - 1)) == 0 ? __ffs(block_size) - 1 : -1) {}
  __device__ __forceinline__ int page(int p) const { return shift >= 0 ? p >> shift : p / size; }
  __device__ __forceinline__ int slot(int p) const { return shift >= 0 ? p & (size - 1) : p % size; }
};

struct CacheView {
  const __bf16* k;
  const __bf16* v;
  const int* table;  // this request's row of the block table
  int table_width;
  PageSize ps;
  int kv_heads, hd, kvh;
  int page0, pages;  // REGS: lane i of `pages` holds the id of page page0 + i of the request
};

// Page id of position p. With REGS the ids of the wave's range were read once, one per lane, and come
// back through a lane shuffle (every lane calls it), so no step waits for a table read before its
// K and V reads can be issued.
template <bool REGS>
__device__ __forceinline__ int page_of(const CacheView& cv, int p) {
  const int index = cv.ps.page(p);
  if (REGS) return __shfl(cv.pages, (index - cv.page0) & 63, 64);
  return cv.table[min(max(index, 0), cv.table_width - 1)];
}

// The K and V^T operands of one step of 32 positions.
struct StepOperands {
  bf16x8 kf[2][KS];  // two 16-row tiles of K: row r of tile t is position kb + 8 (r / 4) + 4 t + r % 4
  bf16x8 vf[DT];     // V^T: positions kb + 8g .. +7 of output dim 16 dt + lr
};

// Issue the loads of the step that starts at kb. No load sits behind a branch (the compiler can then
// count which loads a use waits for, and the next step's stay in flight): a position outside
// [begin, end) reads a position inside it instead, a dim past the head width reads dim 0, a page id
// that is not held reads page 0. None of these can reach a result: such a position's score is masked
// before the softmax and its weight is zero, the query is zero in the padded dims and padded output
// dims are not stored; what is read in their place is cache content of the same request. The group of eight V
// positions that holds `end - 1` may reach past `end`, into slots that this request has not written: the range's
// last step zeroes those elements (keep_before_end). The block table is checked on the host before a step runs.
template <bool REGS>
__device__ __forceinline__ void load_step(int kb, int begin, int end, const CacheView& cv, StepOperands& r) {
  const int lane = threadIdx.x & 63, lr = lane & 15, lg = lane >> 4;
  const int bs = cv.ps.size, hd = cv.hd;
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) {
    const int p = min(max(kb + (lr >> 2) * 8 + sub * 4 + (lr & 3), begin), end - 1);
    const int page = max(page_of<REGS>(cv, p), 0);
    const __bf16* row = cv.k + (((size_t)page * cv.kv_heads + cv.kvh) * bs + cv.ps.slot(p)) * hd;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int dim = ks * 32 + lg * 8;
      r.kf[sub][ks] = *(const bf16x8*)(row + (dim < hd ? dim : 0));
    }
  }
  // groups of eight positions start at multiples of 8 and lie in one page (8 divides the page size)
  const int pv = min(max(kb + lg * 8, begin & ~7), (end - 1) & ~7);
  const int vpage = max(page_of<REGS>(cv, pv), 0);
  const __bf16* vrow = cv.v + (((size_t)vpage * cv.kv_heads + cv.kvh) * hd) * bs + cv.ps.slot(pv);
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int d = dt * 16 + lr;
    r.vf[dt] = *(const bf16x8*)(vrow + (size_t)(d < hd ? d : 0) * bs);
  }
}

// Online-softmax attention of 16 columns over positions [begin, end). Per lane: col_lo / col_pos are
// the visible range [lo, pos] of the lane's column (pos < 0: the column is empty).
// State: o[DT] (O^T tiles), m (running max of the column), l (this lane's share of the running sum).
// The loads of a step are issued one step ahead of its arithmetic (two operand sets that alternate by
// unrolling): a wave has few steps and memory is the bound.
template <bool REGS>
__device__ __forceinline__ void attend_range(const bf16x8 (&qf)[KS], int col_lo, int col_pos, int begin, int end,
                                             const CacheView& cv, float scale, f32x4 (&o)[DT], float& m, float& l) {
  const int lane = threadIdx.x & 63, lg = lane >> 4;
  const int first = begin & ~31;
  if (first >= end) return;
  StepOperands ops[2];
  auto step = [&](auto set_, auto rem_, int i) {
    constexpr int SET = decltype(set_)::value;
    const int kb = first + i * 32;
    if constexpr (decltype(rem_)::value >= 1) load_step<REGS>(kb + 32, begin, end, cv, ops[SET ^ 1]);
    const StepOperands& cur = ops[SET];
    // ---- scores of two 16-position tiles
    f32x4 s[2];
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.kf[sub][ks], qf[ks], acc, 0, 0, 0);
      s[sub] = acc;
    }
    // ---- mask, running max, weights
    float sv[8];
    float tile_max = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int p = kb + lg * 8 + sub * 4 + j;
        const bool visible = p >= col_lo && p <= col_pos && p >= begin && p < end;
        const float x = visible ? s[sub][j] * scale : -INFINITY;
        sv[sub * 4 + j] = x;
        tile_max = fmaxf(tile_max, x);
      }
    tile_max = max_of_column(tile_max);
    const float m_new = fmaxf(m, tile_max);
    float alpha = 1.f;
    bf16x8 pf = zero8();
    if (m_new > -INFINITY) {
      alpha = __expf(m - m_new);  // m = -inf gives 0
      float sum = 0.f;
#pragma unroll
      for (int i8 = 0; i8 < 8; ++i8) {
        const float w = __expf(sv[i8] - m_new);
        sum += w;
        pf[i8] = (__bf16)w;
      }
      l = l * alpha + sum;
      m = m_new;
    }
    // the last step of the range (known when it is compiled): V slots at or past `end` count as zero
    constexpr bool LAST = decltype(rem_)::value == 0;
    const int kept = end - (kb + lg * 8);
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      o[dt] *= alpha;
      const bf16x8 vf = LAST ? keep_before_end(cur.vf[dt], kept, kept - 4) : cur.vf[dt];
      o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf, o[dt], 0, 0, 0);
    }
  };
  load_step<REGS>(first, begin, end, cv, ops[0]);
  run_pipeline<2, 1>(step, (end - first + 31) / 32);
}

__device__ __forceinline__ void load_q(const __bf16* qrow, int hd, bf16x8 (&qf)[KS]) {
  const int lg = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    qf[ks] = (qrow && ks * 32 + lg * 8 < hd) ? *(const bf16x8*)(qrow + ks * 32 + lg * 8) : zero8();
}

// ---------------------------------------------------------------------------------------------
// Prompts: one workgroup of eight waves per (tile, head). A tile is 128 consecutive tokens of one entry; a wave owns
// 16 of them (one block of columns). The positions are walked in tiles of 64 whose K rows and V^T rows
// are fetched once per workgroup into LDS and read from there by all eight waves: while a tile is being
// multiplied the next one's loads are in flight in registers, and the page ids of the tile after that
// are already being looked up. Two workgroups fit a CU, so one's barriers and loads hide behind the
// other's arithmetic. LDS rows are padded by 16 bytes, which spreads the 16 rows of an operand read over
// the banks only in part (such reads measured at 0.7 of the LDS rate). This kernel takes every head width
// and page size; widths of 64, 128 and 256 that fill their padded width, with pages that divide 64, take
// attn_prefill_direct_kernel below, which swizzles instead of padding.
constexpr int PT_WAVES = 8;
constexpr int PT_THREADS = PT_WAVES * 64;
constexpr int PT_TOKENS = PT_WAVES * 16;   // tokens of a tile
constexpr int PT_KV = 64;                  // positions of a K/V tile
constexpr int PT_KROW = HDP + 8;           // elements of a K row in LDS
constexpr int PT_VROW = PT_KV + 8;         // elements of a V^T row in LDS: 144 bytes
constexpr int PT_PIECES = PT_KV * HDP / 8; // 16-byte pieces of a K tile, and of a V^T tile
constexpr int PT_PER_THREAD = (PT_PIECES + PT_THREADS - 1) / PT_THREADS;

template <bool FAST>
__global__ __launch_bounds__(PT_THREADS) void attn_prefill_kernel(
    const __bf16* __restrict__ q, long long q_stride, const __bf16* __restrict__ k_cache,
    const __bf16* __restrict__ v_cache, __bf16* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos,
    const int* __restrict__ block_table, int table_width, int block_size, int heads, int kv_heads, int hd,
    float scale, int window, int cus) {
  extern __shared__ __attribute__((aligned(16))) __bf16 lds[];
  __bf16* sK = lds;                     // [PT_KV][PT_KROW]
  __bf16* sV = lds + PT_KV * PT_KROW;   // [HDP][PT_VROW]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, lr = lane & 15, lg = lane >> 4;
  // Work items (tile, head) are numbered by rising length (the host sorts the tiles). Workgroups are
  // handed out in rounds of one per CU and two share a CU: even rounds take the longest items left,
  // odd rounds the shortest, so that a long tile's neighbour on its CU is a short one.
  const int total = (int)gridDim.x, round = blockIdx.x / cus;
  const int taken = (round >> 1) * cus + blockIdx.x % cus;
  const int item = (round & 1) ? taken : total - 1 - taken;
  const int tile = item / heads;
  const int entry = tiles[2 * tile], tile_off = tiles[2 * tile + 1];
  const int h = item % heads, kvh = h / (heads / kv_heads);
  const int tok0 = entry_start[entry], count = entry_start[entry + 1] - tok0;
  const int first_pos = entry_first_pos[entry];
  const int* table = block_table + (size_t)entry * table_width;
  const int bs = block_size;
  const PageSize ps(block_size);

  // the workgroup's range of positions
  const int tile_cols = min(PT_TOKENS, count - tile_off);
  const int tile_first_pos = first_pos + tile_off;
  const int begin = (window > 0 && tile_first_pos + 1 > window) ? tile_first_pos + 1 - window : 0;
  const int end = tile_first_pos + tile_cols;  // one past the last column's position

  // this wave's columns
  const int q_off = tile_off + wave * 16;
  const int c = q_off + lr;
  const bool col_ok = c < count;
  const int col_pos = col_ok ? first_pos + c : -1;
  const int col_lo = (window > 0 && col_pos + 1 > window) ? col_pos + 1 - window : 0;
  bf16x8 qf[KS];
  load_q(col_ok ? q + (size_t)(tok0 + c) * q_stride + (size_t)h * hd : nullptr, hd, qf);
  const int wave_cols = max(0, min(16, count - q_off));
  const int wave_end = wave_cols > 0 ? first_pos + q_off + wave_cols : 0;  // nothing at or past it is visible
  const int wave_first = first_pos + q_off;
  const int wave_begin = (window > 0 && wave_first + 1 > window) ? wave_first + 1 - window : 0;
  const int wave_last = wave_end - 1;  // position of the wave's last column
  const int wave_lo_max = (window > 0 && wave_last + 1 > window) ? wave_last + 1 - window : 0;

  f32x4 o[DT];
  float m = -INFINITY, l = 0.f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // per thread: PT_PER_THREAD pieces of the K tile (row r, 8 dims) and of the V^T tile (dim d, 8 positions)
  bf16x8 k_stage[PT_PER_THREAD], v_stage[PT_PER_THREAD];
  int k_page[PT_PER_THREAD], v_page[PT_PER_THREAD];
  // FAST: the page size is a power of two that divides 64. Tiles start at multiples of 64, so which page of
  // a tile a piece lies in, and where in that page, is the same for every tile: the thread keeps both, a tile's
  // page id is one table read at a clamped index, and an address is one multiply-add. Nothing is loaded
  // conditionally: a piece outside [begin, end) reads a page of the same request inside that range, and its
  // positions are masked, or weigh zero, for every column; the V^T operands of the tile that holds `end` are
  // zeroed from `end` on (keep_before_end), since the slots there may hold anything.
  int k_tab[PT_PER_THREAD], v_tab[PT_PER_THREAD];          // page of the piece within a tile
  unsigned k_in[PT_PER_THREAD], v_in[PT_PER_THREAD];       // byte offset of the piece within its page
  const unsigned page_bytes = (unsigned)(kv_heads * bs * hd * 2);
  const int page_lo = ps.page(begin), page_hi = ps.page(end - 1);
  if constexpr (FAST) {
#pragma unroll
    for (int i = 0; i < PT_PER_THREAD; ++i) {
      const int id = min(tid + PT_THREADS * i, PT_PIECES - 1);
      const int r = id / (HDP / 8), ck = id % (HDP / 8);
      k_tab[i] = r >> ps.shift;
      k_in[i] = (unsigned)((((kvh * bs + (r & (bs - 1))) * hd) + min(ck * 8, hd - 8)) * 2);
      const int d = id / (PT_KV / 8), cv = id % (PT_KV / 8);
      v_tab[i] = (cv * 8) >> ps.shift;
      v_in[i] = (unsigned)((((kvh * hd + min(d, hd - 1)) * bs) + ((cv * 8) & (bs - 1))) * 2);
    }
  }
  auto lookup = [&](int p0) {  // page ids of the tile at p0 (without FAST, -1: nothing to read)
    if constexpr (FAST) {
      const int tp = p0 >> ps.shift;
#pragma unroll
      for (int i = 0; i < PT_PER_THREAD; ++i) {
        k_page[i] = table[min(max(tp + k_tab[i], page_lo), page_hi)];
        v_page[i] = table[min(max(tp + v_tab[i], page_lo), page_hi)];
      }
    } else {
#pragma unroll
      for (int i = 0; i < PT_PER_THREAD; ++i) {
        const int id = tid + PT_THREADS * i;
        const int pk = p0 + id / (HDP / 8);
        k_page[i] = (id < PT_PIECES && pk >= begin && pk < end) ? table[ps.page(pk)] : -1;
        const int pv = p0 + (id % (PT_KV / 8)) * 8;  // eight positions of one page (8 divides the page size)
        v_page[i] = (id < PT_PIECES && pv + 7 >= begin && pv < end) ? table[ps.page(pv)] : -1;
      }
    }
  };
  auto fetch = [&](int p0) {
    if constexpr (FAST) {
#pragma unroll
      for (int i = 0; i < PT_PER_THREAD; ++i) {
        k_stage[i] = *(const bf16x8*)((const char*)k_cache + ((size_t)(unsigned)k_page[i] * page_bytes + k_in[i]));
        v_stage[i] = *(const bf16x8*)((const char*)v_cache + ((size_t)(unsigned)v_page[i] * page_bytes + v_in[i]));
      }
    } else {
#pragma unroll
      for (int i = 0; i < PT_PER_THREAD; ++i) {
        const int id = tid + PT_THREADS * i;
        const int r = id / (HDP / 8), ck = id % (HDP / 8);
        const int pk = p0 + r;
        k_stage[i] = (k_page[i] >= 0 && ck * 8 < hd)
                         ? *(const bf16x8*)(k_cache + (((size_t)k_page[i] * kv_heads + kvh) * bs + ps.slot(pk)) * hd + ck * 8)
                         : zero8();
        const int d = id / (PT_KV / 8), cv = id % (PT_KV / 8);
        const int pv = p0 + cv * 8;
        v_stage[i] = (v_page[i] >= 0 && d < hd)
                         ? *(const bf16x8*)(v_cache + (((size_t)v_page[i] * kv_heads + kvh) * hd + d) * bs + ps.slot(pv))
                         : zero8();
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < PT_PER_THREAD; ++i) {
      const int id = tid + PT_THREADS * i;
      if (id < PT_PIECES) {
        *(bf16x8*)(sK + (id / (HDP / 8)) * PT_KROW + (id % (HDP / 8)) * 8) = k_stage[i];
        // Within each group of 32 positions a V^T row is stored in the order in which the weights sit in
        // the matrix instruction's operand: four positions of one 16-position tile, then the four at the
        // same place in the next tile. A lane's operand is then one 16-byte read. A piece of 8 positions
        // goes in as two halves, 16 bytes apart.
        const int cv8 = (id % (PT_KV / 8)) * 8;   // first position of the piece within the tile
        __bf16* dst_v = sV + (id / (PT_KV / 8)) * PT_VROW + (cv8 & 32) + ((cv8 & 8) ? 16 : 0) + ((cv8 & 16) ? 4 : 0);
        bf16x4 lo, hi;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          lo[j] = v_stage[i][j];
          hi[j] = v_stage[i][4 + j];
        }
        *(bf16x4*)dst_v = lo;
        *(bf16x4*)(dst_v + 8) = hi;
      }
    }
  };

  // One tile of 64 positions for this wave's 16 columns. The running maximum m is kept in units of the raw
  // score (the scale is positive, so it commutes with the maximum) and a weight is one fused multiply-add
  // and one exp2: exp2(s * c - m * c) with c = scale * log2(e). `masked`: some column of the wave does not
  // see all 64 positions (the tiles on the diagonal and at a window's edge); the other tiles skip the
  // comparisons. The sums are rescaled only when some column's maximum moved, which is rare after the
  // first tiles.
  const float c2 = scale * 1.44269504088896341f;
  auto tile_body = [&](bool masked, int p0) {
    // ---- scores of four 16-position tiles
    f32x4 s[4];
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 kf = *(const bf16x8*)(sK + (sub * 16 + lr) * PT_KROW + ks * 32 + lg * 8);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], acc, 0, 0, 0);
      }
      s[sub] = acc;
    }
    // ---- mask, running max, weights
    if (masked) {
#pragma unroll
      for (int sub = 0; sub < 4; ++sub)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int p = p0 + sub * 16 + lg * 4 + j;
          if (!(p >= col_lo && p <= col_pos)) s[sub][j] = -INFINITY;
        }
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 4; ++sub)
#pragma unroll
      for (int j = 0; j < 4; ++j) tile_max = fmaxf(tile_max, s[sub][j]);
    tile_max = max_of_column(tile_max);
    const float m_new = fmaxf(m, tile_max);
    bf16x8 pf[2] = {zero8(), zero8()};
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
      const float alpha = (m_new > m && m > -INFINITY) ? __builtin_amdgcn_exp2f((m - m_new) * c2) : 1.f;
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] *= alpha;
      m = m_new;
    }
    if (m_new > -INFINITY) {   // a masked tile may hold nothing for this column yet
      const float mc = m_new * c2;
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float w = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i >> 2][i & 3], c2, -mc));
        sum += w;
        pf[i >> 3][i & 7] = (__bf16)w;   // step 0: tiles 0 and 1; step 1: tiles 2 and 3
      }
      l += sum;
    }
    // ---- output: V^T operands from LDS (elements 0-3: positions 4 lg .. of a step's first 16, 4-7: of its second 16)
    const bool tail = p0 + PT_KV > end;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int step = 0; step < 2; ++step) {
        bf16x8 vf = *(const bf16x8*)(sV + (dt * 16 + lr) * PT_VROW + step * 32 + lg * 8);
        if (tail) {
          const int kept = end - (p0 + step * 32 + lg * 4);
          vf = keep_before_end(vf, kept, kept - 16);
        }
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[step], o[dt], 0, 0, 0);
      }
    }
  };

  const int first_tile = begin & ~(PT_KV - 1);
  lookup(first_tile);
  fetch(first_tile);
  lookup(first_tile + PT_KV);
  stash();
  __syncthreads();
  for (int p0 = first_tile; p0 < end; p0 += PT_KV) {
    const bool more = p0 + PT_KV < end;
    if (more) {
      fetch(p0 + PT_KV);        // with the page ids looked up one tile ago
      lookup(p0 + 2 * PT_KV);
    }
    if (p0 < wave_end && p0 + PT_KV > wave_begin)   // some of this tile is visible to this wave
      tile_body(!(p0 + PT_KV - 1 <= wave_first && p0 >= wave_lo_max), p0);
    __syncthreads();  // everyone is done with this tile
    if (more) {
      stash();
      __syncthreads();
    }
  }
  l = sum_of_column(l);
  if (!col_ok) return;
  const float inv = 1.f / l;
  __bf16* dst = out + (size_t)(tok0 + c) * heads * hd + (size_t)h * hd;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int d = dt * 16 + lg * 4;
    if (d < hd) {
      bf16x4 r;
#pragma unroll
      for (int j = 0; j < 4; ++j) r[j] = (__bf16)(o[dt][j] * inv);
      *(bf16x4*)(dst + d) = r;
    }
  }
}

// ---------------------------------------------------------------------------------------------
// The prompt kernel for head widths of 64, 128 and 256 that fill their padded width, and page sizes that are
// powers of two dividing 64: K and V^T tiles go from the cache straight into LDS (loads with the lds modifier:
// no staging registers, no LDS stores) into one of two stages, so that a tile costs one barrier and the next
// tile's loads run under this tile's arithmetic. A load instruction fills 1 KB of LDS, lane L the 16 bytes at
// 16 L, so rows cannot be padded against bank conflicts; instead the 16-byte chunk c of row r sits in slot
// c ^ f(r), the loading lane fetching the chunk that belongs in its slot, with f chosen so that the 16 rows
// which the lanes of an operand read touch different banks. Which position an instruction's K row holds is free
// (every lane reads its own row), and as in the decode kernel row 4g + j of tile t of a 32-position step is
// position 8g + 4t + j: a lane's eight weights are then eight consecutive positions and its V^T operand one
// 16-byte chunk of a V^T row that is stored as it lies in the cache.
//
// SPLIT: a workgroup of sixteen waves, one per CU; waves 0-7 walk the first half of the tile's positions and
// waves 8-15 the second half for the same 128 columns, each half with LDS stages of its own, and the halves'
// (max, sum, weighted sum) are merged through LDS at the end. For a step with few work items of very different
// lengths (one long prompt): a CU then works on its longest item with all sixteen waves instead of being left
// with one workgroup of eight once the short neighbour has finished.
//
// CHUNKED (not with SPLIT): grid (tiles x heads x max_chunks); a tile's 64-position steps are cut into chunks of
// `chunk_tiles`, a workgroup of eight waves takes one chunk (one that the tile does not have ends at once), and
// where a tile has more than one chunk the workgroups leave (max, sum, weighted sum) of their columns in `partial`,
// [tile, head, chunk, 128 columns, hd + 4] floats, for attn_prefill_merge_kernel to merge in ascending order. For a
// model of few heads, whose (tile, head) items are fewer than the CUs and as long as their prompts: the 1.5B shape
// has 12 heads, and four portions of 512 tokens are 192 items of which the one deepest in its prompt sets the time.
#if HDP == 64 || HDP == 128 || HDP == 256
#define VK_PREFILL_DIRECT 1
constexpr int PD_ROWB = HDP * 2;                        // bytes of a K row in LDS
constexpr int PD_C = HDP / 8;                           // 16-byte chunks of a K row
constexpr int PD_KBYTES = PT_KV * PD_ROWB;              // K tile: 64 rows
constexpr int PD_VBYTES = HDP * 128;                    // V^T tile: HDP rows of 64 positions
constexpr int PD_STAGE = PD_KBYTES + PD_VBYTES;
constexpr int PD_KLOADS = PD_KBYTES / 1024 / PT_WAVES;  // load instructions per wave and tile
constexpr int PD_VLOADS = PD_VBYTES / 1024 / PT_WAVES;
constexpr int PD_ROWS_PER_LOAD = 1024 / PD_ROWB;
constexpr bool PD_CAN_SPLIT = 4 * PD_STAGE <= 128 * 1024;  // two halves with two stages each

// slot = chunk ^ k_swizzle(row). The lanes lr = 0..15 of an operand read rows 8 (lr / 4) + lr % 4 (+ a constant):
// with rows of 256 or 512 bytes every row starts at bank 0 and lr itself separates them; rows of 128 bytes
// alternate between the two halves of the banks with lr % 2 and lr % 8 does.
__device__ __forceinline__ int k_swizzle(int r) {
  return PD_C == 8 ? ((((r >> 3) & 1) << 2) | (r & 3)) : ((((r >> 3) & 3) << 2) | (r & 3));
}

constexpr int PD_PARTIAL_ROW = HDP + 4;   // floats of a column's partial result: the weighted sum, max, sum, and padding to 16 bytes

template <bool SPLIT, bool CHUNKED = false>
__global__ __launch_bounds__(SPLIT ? 2 * PT_THREADS : PT_THREADS) void attn_prefill_direct_kernel(
    const __bf16* __restrict__ q, long long q_stride, const __bf16* __restrict__ k_cache,
    const __bf16* __restrict__ v_cache, __bf16* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos,
    const int* __restrict__ block_table, int table_width, int block_size, int heads, int kv_heads, float scale,
    int window, int cus, float* __restrict__ partial, int chunk_tiles, int max_chunks) {
  static_assert(!(SPLIT && CHUNKED), "a chunk is taken by a workgroup of eight waves");
  typedef __attribute__((address_space(3))) void* lds_ptr;
  typedef __attribute__((address_space(1))) const void* global_ptr;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];  // [2][K tile | V^T tile]
  constexpr int hd = HDP;
  const int tid = threadIdx.x, lane = tid & 63, lr = lane & 15, lg = lane >> 4;
  const int wave_of_group = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int half = SPLIT ? wave_of_group >> 3 : 0, wave = SPLIT ? wave_of_group & 7 : wave_of_group;
  unsigned char* lds_half = lds_raw + half * 2 * PD_STAGE;
  // work items as in attn_prefill_kernel: long ones first, paired with short ones on a CU (SPLIT: one
  // workgroup per CU, longest first)
  const int total = CHUNKED ? (int)gridDim.x / max_chunks : (int)gridDim.x, round = blockIdx.x / cus;
  // Workgroups go to the XCDs in turn, and the query heads of one key head read the same K and V: of every 8 x
  // group workgroups in a row the ones that land on one XCD take the heads of one group, so that the XCD's L2
  // fetches those tiles once (with numbers in a row, every head of a group ran on another XCD). Every other run
  // of 8 groups is dealt to the XCDs in the opposite order: the items come sorted by length, and dealt one way
  // only the first XCDs would get the longer item of every run.
  const int heads_per_key = heads / kv_heads;
  auto by_xcd = [&](int number, int count) {
    const int block = 8 * heads_per_key;
    if (number >= count / block * block) return number;
    const int within = number % block;
    const int xcd = ((number / block) & 1) ? 7 - within % 8 : within % 8;
    return number - within + xcd * heads_per_key + within / 8;
  };
  const int taken = (round >> 1) * cus + by_xcd((int)blockIdx.x % cus, min(cus, total - round * cus));
  // CHUNKED: the chunks of one (tile, head) are neighbours, the tiles that see most positions come first
  const int chunk = CHUNKED ? (int)blockIdx.x % max_chunks : 0;
  const int item = CHUNKED ? total - 1 - (int)blockIdx.x / max_chunks
                           : SPLIT ? total - 1 - by_xcd((int)blockIdx.x, total) : (round & 1) ? taken : total - 1 - taken;
  const int tile = item / heads;
  const int entry = tiles[2 * tile], tile_off = tiles[2 * tile + 1];
  const int h = item % heads, kvh = h / (heads / kv_heads);
  const int tok0 = entry_start[entry], count = entry_start[entry + 1] - tok0;
  const int first_pos = entry_first_pos[entry];
  const int* table = block_table + (size_t)entry * table_width;
  const int bs = block_size;
  const PageSize ps(block_size);

  const int tile_cols = min(PT_TOKENS, count - tile_off);
  const int tile_first_pos = first_pos + tile_off;
  const int begin = (window > 0 && tile_first_pos + 1 > window) ? tile_first_pos + 1 - window : 0;
  const int end = tile_first_pos + tile_cols;
  const int first_tile = begin & ~(PT_KV - 1);
  const int all_tiles = (end - first_tile + PT_KV - 1) / PT_KV;
  const int chunks = CHUNKED ? (all_tiles + chunk_tiles - 1) / chunk_tiles : 1;
  if (CHUNKED && chunk >= chunks) return;   // the whole workgroup, before any barrier

  const int q_off = tile_off + wave * 16;
  const int c = q_off + lr;
  const bool col_ok = c < count;
  const int col_pos = col_ok ? first_pos + c : -1;
  const int col_lo = (window > 0 && col_pos + 1 > window) ? col_pos + 1 - window : 0;
  bf16x8 qf[KS];
  load_q(col_ok ? q + (size_t)(tok0 + c) * q_stride + (size_t)h * hd : nullptr, hd, qf);
  const int wave_cols = max(0, min(16, count - q_off));
  const int wave_end = wave_cols > 0 ? first_pos + q_off + wave_cols : 0;
  const int wave_first = first_pos + q_off;
  const int wave_begin = (window > 0 && wave_first + 1 > window) ? wave_first + 1 - window : 0;
  const int wave_last = wave_end - 1;
  const int wave_lo_max = (window > 0 && wave_last + 1 > window) ? wave_last + 1 - window : 0;

  f32x4 o[DT];
  float m = -INFINITY, l = 0.f;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Per lane and load instruction: which page of a tile its chunk lies in and where in that page; both are the
  // same for every tile, since tiles start at multiples of 64 and the page size divides 64. Nothing is loaded
  // conditionally: a chunk outside [begin, end) reads a page of the same request inside that range, and its
  // positions are masked, or weigh zero, for every column; the V^T operands of the tile that holds `end` are
  // zeroed from `end` on (keep_before_end), since the slots there may hold anything.
  int k_tab[PD_KLOADS], v_tab[PD_VLOADS];
  unsigned k_in[PD_KLOADS], v_in[PD_VLOADS];
  const unsigned page_bytes = (unsigned)(kv_heads * bs * hd * 2);
  const int page_lo = ps.page(begin), page_hi = ps.page(end - 1);
#pragma unroll
  for (int i = 0; i < PD_KLOADS; ++i) {
    const int r = (wave * PD_KLOADS + i) * PD_ROWS_PER_LOAD + lane / PD_C;
    const int chunk = (lane % PD_C) ^ k_swizzle(r);
    k_tab[i] = r >> ps.shift;
    k_in[i] = (unsigned)(((kvh * bs + (r & (bs - 1))) * hd + chunk * 8) * 2);
  }
#pragma unroll
  for (int i = 0; i < PD_VLOADS; ++i) {
    const int d = (wave * PD_VLOADS + i) * 8 + (lane >> 3);
    const int p8 = ((lane & 7) ^ (d & 7)) * 8;  // first of the chunk's eight positions within the tile
    v_tab[i] = p8 >> ps.shift;
    v_in[i] = (unsigned)(((kvh * hd + d) * bs + (p8 & (bs - 1))) * 2);
  }
  int k_page[PD_KLOADS], v_page[PD_VLOADS];
  auto lookup = [&](int p0) {
    const int tp = p0 >> ps.shift;
#pragma unroll
    for (int i = 0; i < PD_KLOADS; ++i) k_page[i] = table[min(max(tp + k_tab[i], page_lo), page_hi)];
#pragma unroll
    for (int i = 0; i < PD_VLOADS; ++i) v_page[i] = table[min(max(tp + v_tab[i], page_lo), page_hi)];
  };
  auto issue = [&](int stage) {
    unsigned char* to_k = lds_half + stage * PD_STAGE + wave * PD_KLOADS * 1024;
    unsigned char* to_v = lds_half + stage * PD_STAGE + PD_KBYTES + wave * PD_VLOADS * 1024;
#pragma unroll
    for (int i = 0; i < PD_KLOADS; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_ptr)((const char*)k_cache + ((size_t)(unsigned)k_page[i] * page_bytes + k_in[i])),
          (lds_ptr)(to_k + i * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < PD_VLOADS; ++i)
      __builtin_amdgcn_global_load_lds(
          (global_ptr)((const char*)v_cache + ((size_t)(unsigned)v_page[i] * page_bytes + v_in[i])),
          (lds_ptr)(to_v + i * 1024), 16, 0, 0);
  };

  // a lane's operand addresses within a stage
  const int fk = PD_C == 8 ? (lr & 7) : lr;
  unsigned k_at[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks)
    k_at[ks] = (unsigned)((8 * (lr >> 2) + (lr & 3)) * PD_ROWB + (((ks * 4 + lg) ^ fk) * 16));
  unsigned v_at[2];
#pragma unroll
  for (int st = 0; st < 2; ++st)
    v_at[st] = (unsigned)(PD_KBYTES + lr * 128 + (((st * 4 + lg) ^ (lr & 7)) * 16));

  const float c2 = scale * 1.44269504088896341f;
  auto tile_body = [&](bool masked, int p0, const unsigned char* base) {
    // ---- scores: tile sub = 2 st + t holds positions p0 + 32 st + 8 g + 4 t + j in register j of lane group g
    f32x4 s[4];
#pragma unroll
    for (int sub = 0; sub < 4; ++sub) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        const bf16x8 kf = *(const bf16x8*)(base + k_at[ks] + ((sub >> 1) * 32 + (sub & 1) * 4) * PD_ROWB);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf, qf[ks], acc, 0, 0, 0);
      }
      s[sub] = acc;
    }
    if (masked) {
#pragma unroll
      for (int sub = 0; sub < 4; ++sub)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int p = p0 + (sub >> 1) * 32 + lg * 8 + (sub & 1) * 4 + j;
          if (!(p >= col_lo && p <= col_pos)) s[sub][j] = -INFINITY;
        }
    }
    float tile_max = -INFINITY;
#pragma unroll
    for (int sub = 0; sub < 4; ++sub)
#pragma unroll
      for (int j = 0; j < 4; ++j) tile_max = fmaxf(tile_max, s[sub][j]);
    tile_max = max_of_column(tile_max);
    const float m_new = fmaxf(m, tile_max);
    if (__builtin_amdgcn_ballot_w64(m_new > m) != 0) {
      const float alpha = (m_new > m && m > -INFINITY) ? __builtin_amdgcn_exp2f((m - m_new) * c2) : 1.f;
      l *= alpha;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) o[dt] *= alpha;
      m = m_new;
    }
    // No branch around the weights: a column that sees nothing yet has m = -inf and only masked scores, which
    // give exp2(-inf - 0) = 0, as a masked score under a finite m does.
    bf16x8 pf[2];
    {
      const float mc = m_new > -INFINITY ? m_new * c2 : 0.f;
      float sum = 0.f;
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float w = __builtin_amdgcn_exp2f(__builtin_fmaf(s[i >> 2][i & 3], c2, -mc));
        sum += w;
        pf[i >> 3][i & 7] = (__bf16)w;  // step st: tiles 2 st and 2 st + 1, eight consecutive positions
      }
      l += sum;
    }
    const bool tail = p0 + PT_KV > end;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
      for (int st = 0; st < 2; ++st) {
        bf16x8 vf = *(const bf16x8*)(base + v_at[st] + dt * 16 * 128);
        if (tail) {
          const int kept = end - (p0 + st * 32 + lg * 8);
          vf = keep_before_end(vf, kept, kept - 4);
        }
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf, pf[st], o[dt], 0, 0, 0);
      }
    }
  };

  // this half's tiles: all of them, or with SPLIT the first or the second half of them (both halves pass the
  // same number of barriers)
  const int steps = CHUNKED ? min(chunk_tiles, all_tiles - chunk * chunk_tiles) : SPLIT ? (all_tiles + 1) / 2 : all_tiles;
  const int my_tiles = half ? all_tiles - steps : steps;
  const int my_first = first_tile + (CHUNKED ? chunk * chunk_tiles * PT_KV : half ? steps * PT_KV : 0);
  lookup(my_first);
  if (my_tiles > 0) issue(0);
  lookup(my_first + PT_KV);
  wait_own_loads();
  __syncthreads();
  int stage = 0;
  for (int i = 0; i < steps; ++i) {
    const int p0 = my_first + i * PT_KV;
    if (i + 1 < my_tiles) {
      issue(stage ^ 1);            // nobody reads that stage any more: the barrier that ended the last tile
      lookup(p0 + 2 * PT_KV);
    }
    if (i < my_tiles && p0 < wave_end && p0 + PT_KV > wave_begin)
      tile_body(!(p0 + PT_KV - 1 <= wave_first && p0 >= wave_lo_max), p0, lds_half + stage * PD_STAGE);
    wait_own_loads();   // a barrier alone does not wait for loads that write LDS
    __syncthreads();
    stage ^= 1;
  }
  if constexpr (SPLIT) {
    // the second half hands its state over in LDS (every tile has been read: the loop's last barrier)
    f32x4* hand_o = (f32x4*)lds_raw;                                        // [8 waves][DT][64 lanes]
    float* hand_ml = (float*)(lds_raw + PT_WAVES * DT * 64 * sizeof(f32x4));  // [8 waves][64 lanes][m, l]
    if (half) {
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) hand_o[(wave * DT + dt) * 64 + lane] = o[dt];
      hand_ml[(wave * 64 + lane) * 2] = m;
      hand_ml[(wave * 64 + lane) * 2 + 1] = l;
    }
    __syncthreads();
    if (half) return;
    const float m1 = hand_ml[(wave * 64 + lane) * 2], l1 = hand_ml[(wave * 64 + lane) * 2 + 1];
    const float m_both = fmaxf(m, m1);
    const float a0 = m > -INFINITY ? __builtin_amdgcn_exp2f((m - m_both) * c2) : 0.f;
    const float a1 = m1 > -INFINITY ? __builtin_amdgcn_exp2f((m1 - m_both) * c2) : 0.f;
    l = l * a0 + l1 * a1;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) o[dt] = o[dt] * a0 + hand_o[(wave * DT + dt) * 64 + lane] * a1;
  }
  l = sum_of_column(l);
  if (!col_ok) return;
  if (CHUNKED && chunks > 1) {  // a column that sees nothing of this chunk leaves a maximum of -inf and sums of zero
    float* dst = partial + ((((size_t)tile * heads + h) * max_chunks + chunk) * PT_TOKENS + (wave * 16 + lr)) * PD_PARTIAL_ROW;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) *(f32x4*)(dst + dt * 16 + lg * 4) = o[dt];
    if (lg == 0) {
      dst[hd] = m;
      dst[hd + 1] = l;
    }
    return;
  }
  const float inv = 1.f / l;
  __bf16* dst = out + (size_t)(tok0 + c) * heads * hd + (size_t)h * hd;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    bf16x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = (__bf16)(o[dt][j] * inv);
    *(bf16x4*)(dst + dt * 16 + lg * 4) = r;
  }
}

// The chunks of attn_prefill_direct_kernel<false, true> merged: grid (tiles, heads, 128 * HDP / 4 / 256), a thread
// four dims of one column. The maxima are raw scores (the kernel scales inside its exponentials); the chunks are
// folded in ascending order, acc = acc 2^((M - M') c) + acc_c 2^((m_c - M') c) with M' the larger of the running
// maximum M and m_c, the sums likewise, four chunks requested at a time. A tile of one chunk was written by the
// kernel itself.
__global__ __launch_bounds__(256) void attn_prefill_merge_kernel(const float* __restrict__ partial, __bf16* __restrict__ out,
                                                                 const int* __restrict__ tiles,
                                                                 const int* __restrict__ entry_start,
                                                                 const int* __restrict__ entry_first_pos, int heads,
                                                                 float scale, int window, int chunk_tiles, int max_chunks) {
  constexpr int hd = HDP, QUADS = HDP / 4, AHEAD = 4;
  const int tile = blockIdx.x, h = blockIdx.y;
  const int entry = tiles[2 * tile], tile_off = tiles[2 * tile + 1];
  const int tok0 = entry_start[entry], count = entry_start[entry + 1] - tok0;
  const int tile_cols = min(PT_TOKENS, count - tile_off);
  const int tile_first_pos = entry_first_pos[entry] + tile_off;
  const int begin = (window > 0 && tile_first_pos + 1 > window) ? tile_first_pos + 1 - window : 0;
  const int end = tile_first_pos + tile_cols;
  const int first_tile = begin & ~(PT_KV - 1);
  const int all_tiles = (end - first_tile + PT_KV - 1) / PT_KV;
  const int chunks = (all_tiles + chunk_tiles - 1) / chunk_tiles;
  if (chunks <= 1) return;
  const int at = blockIdx.z * 256 + threadIdx.x;
  const int col = at / QUADS, quad = at % QUADS;
  if (col >= tile_cols) return;
  const float c2 = scale * 1.44269504088896341f;
  const size_t chunk_stride = (size_t)PT_TOKENS * PD_PARTIAL_ROW;
  const float* of_col = partial + ((size_t)tile * heads + h) * max_chunks * chunk_stride + (size_t)col * PD_PARTIAL_ROW;
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  float total = 0.f, best = -INFINITY;
  for (int ch0 = 0; ch0 < chunks; ch0 += AHEAD) {
    float mc[AHEAD], lc[AHEAD];
    f32x4 oc[AHEAD];
#pragma unroll
    for (int j = 0; j < AHEAD; ++j) {   // a clamped chunk is not folded in
      const float* src = of_col + (size_t)min(ch0 + j, chunks - 1) * chunk_stride;
      mc[j] = src[hd];
      lc[j] = src[hd + 1];
      oc[j] = *(const f32x4*)(src + quad * 4);
    }
#pragma unroll
    for (int j = 0; j < AHEAD; ++j)
      if (ch0 + j < chunks && mc[j] > -INFINITY) {
        const float both = fmaxf(best, mc[j]);
        const float keep = best > -INFINITY ? __builtin_amdgcn_exp2f((best - both) * c2) : 0.f;
        const float take = __builtin_amdgcn_exp2f((mc[j] - both) * c2);
        acc = acc * keep + oc[j] * take;
        total = total * keep + lc[j] * take;
        best = both;
      }
  }
  const float inv = 1.f / total;
  bf16x4 r;
#pragma unroll
  for (int j = 0; j < 4; ++j) r[j] = (__bf16)(acc[j] * inv);
  *(bf16x4*)(out + (size_t)(tok0 + tile_off + col) * heads * hd + (size_t)h * hd + quad * 4) = r;
}
#endif

// ---------------------------------------------------------------------------------------------
// Decoding: grid (entries, kv_heads * head_blocks, chunks), one wave. Columns are the query heads of
// one key head. Chunk c covers positions [c * chunk, (c + 1) * chunk) of the visible range and leaves
// (max, sum, weighted sum) in `partial`: [entry, head, chunk, hd + 2] floats. REGS: a chunk spans at most
// 64 pages, whose ids the wave reads once.
// JOINED: grid (entries, kv_heads * head_blocks), a workgroup of `chunks` waves (at most JOINED_WAVES), wave c
// taking chunk c; the waves leave (max, sum, weighted sum) in LDS and merge them there, wave w the output tiles
// w, w + chunks, ... in ascending order of the chunks, and write `out` themselves: no `partial`, no second kernel.
// For steps whose (entry, key head) pairs alone fill the GPU (64 requests x 4 key heads), where the chunks only
// serve to keep several waves on a CU.
constexpr int JOINED_WAVES = 8;
// Waves per SIMD that the kernel's registers are sized for: two (256 registers a lane); with a head width of 256 the
// output sums and the operands in flight take more than that and would spill some 400 values, so one.
#if HDP > 128
#define VK_DECODE_WAVES_PER_SIMD 1
#else
#define VK_DECODE_WAVES_PER_SIMD 2
#endif
template <bool REGS, bool JOINED>
__global__ __launch_bounds__(JOINED ? JOINED_WAVES * 64 : 64) __attribute__((amdgpu_waves_per_eu(VK_DECODE_WAVES_PER_SIMD))) void attn_decode_kernel(
    const __bf16* __restrict__ q, long long q_stride, const __bf16* __restrict__ k_cache,
    const __bf16* __restrict__ v_cache, float* __restrict__ partial, __bf16* __restrict__ out,
    const int* __restrict__ entries, const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos,
    const int* __restrict__ block_table, int table_width, int block_size, int heads, int kv_heads, int hd,
    float scale, int window, int chunk, int head_blocks, int dense) {
  const int lane = threadIdx.x & 63, lr = lane & 15, lg = lane >> 4;
  const int wave = JOINED ? __builtin_amdgcn_readfirstlane(threadIdx.x >> 6) : 0;
  const int chunk_index = JOINED ? wave : blockIdx.z, chunks = JOINED ? (int)(blockDim.x >> 6) : (int)gridDim.z;
  // dense: entry i is slot i and holds token i (a step of single tokens only), which saves two reads that the
  // position, and with it every other read, would wait for
  const int slot = blockIdx.x, entry = dense ? slot : entries[slot];
  const int kvh = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int group = heads / kv_heads;
  const int token = dense ? slot : entry_start[entry];
  const PageSize ps(block_size);
  // without a window a chunk's first page does not depend on the position: its page ids are asked for beside it
  int early_pages = -1;
  if (REGS && window == 0)
    early_pages = block_table[(size_t)entry * table_width + min(ps.page(chunk_index * chunk) + lane, table_width - 1)];
  const int pos = entry_first_pos[entry];
  const int lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int begin = max(lo, chunk_index * chunk), end = min(pos + 1, (chunk_index + 1) * chunk);
  const int head_in_group = hb * 16 + lr;
  const bool col_ok = head_in_group < group;
  const int h = kvh * group + head_in_group;
  float* dst = partial + (((size_t)slot * heads + (col_ok ? h : 0)) * chunks + chunk_index) * (hd + 2);
  f32x4 o[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) o[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  if (begin >= end) {  // nothing of this chunk is visible
    if constexpr (!JOINED) {
      if (col_ok && lg == 0) {
        dst[hd] = -INFINITY;
        dst[hd + 1] = 0.f;
      }
      return;
    }
  } else {
    bf16x8 qf[KS];
    load_q(col_ok ? q + (size_t)token * q_stride + (size_t)h * hd : nullptr, hd, qf);
    CacheView cv{k_cache, v_cache, block_table + (size_t)entry * table_width, table_width, ps,
                 kv_heads, hd, kvh, ps.page(begin), early_pages};
    if (REGS && window != 0) {
      const int index = cv.page0 + lane;
      if (index <= ps.page(end - 1) && index < table_width) cv.pages = cv.table[index];
    }
    attend_range<REGS>(qf, lo, col_ok ? pos : -1, begin, end, cv, scale, o, m, l);
    l = sum_of_column(l);
  }
  if constexpr (JOINED) {
    extern __shared__ __attribute__((aligned(16))) float joined_lds[];
    f32x4* sums = (f32x4*)joined_lds;                              // [chunks][DT][64]
    float* max_sum = joined_lds + (size_t)chunks * DT * 64 * 4;    // [chunks][16][2]
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) sums[(wave * DT + dt) * 64 + lane] = o[dt];
    if (lg == 0) {
      max_sum[(wave * 16 + lr) * 2] = m;
      max_sum[(wave * 16 + lr) * 2 + 1] = l;
    }
    __syncthreads();
    // out = sum_c acc_c e^(m_c - M) / sum_c l_c e^(m_c - M) with M = max m_c, as attn_combine_kernel merges
    float best = -INFINITY;
    for (int c = 0; c < chunks; ++c) best = fmaxf(best, max_sum[(c * 16 + lr) * 2]);
    float total = 0.f;
    for (int c = 0; c < chunks; ++c) {
      const float mc = max_sum[(c * 16 + lr) * 2];
      total += (mc > -INFINITY ? __expf(mc - best) : 0.f) * max_sum[(c * 16 + lr) * 2 + 1];
    }
    const float inv = 1.f / total;
    for (int dt = wave; dt < DT; dt += chunks) {
      f32x4 acc = {0.f, 0.f, 0.f, 0.f};
      for (int c = 0; c < chunks; ++c) {
        const float mc = max_sum[(c * 16 + lr) * 2];
        if (mc > -INFINITY) acc += sums[(c * DT + dt) * 64 + lane] * __expf(mc - best);   // an empty chunk adds nothing
      }
      const int d = dt * 16 + lg * 4;
      if (col_ok && d < hd) {
        bf16x4 r;
#pragma unroll
        for (int j = 0; j < 4; ++j) r[j] = (__bf16)(acc[j] * inv);
        *(bf16x4*)(out + (size_t)token * heads * hd + (size_t)h * hd + d) = r;
      }
    }
    return;
  }
  if (!col_ok) return;
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) {
    const int d = dt * 16 + lg * 4;
    if (d < hd) *(f32x4*)(dst + d) = o[dt];
  }
  if (lg == 0) {
    dst[hd] = m;
    dst[hd + 1] = l;
  }
}

// Merge the chunks of one (entry, head): M = max m_c; out = sum_c acc_c e^(m_c - M) / sum_c l_c e^(m_c - M)
// (layer.cu:443-467). One workgroup of four waves per (entry, head). The kernel is a few memory round trips long
// and nothing else, so everything it reads is requested at its start, before anything is computed: the token's
// row, the chunks' (max, sum), and of the weighted sums the first four chunks of every thread, which with up to
// 4 * parts chunks is all of them. Thread -> (part, four output dims); part p sums the chunks p, p + parts, ...
// in ascending order, and the parts are added in ascending order: one fixed order for a given head width and
// number of chunks.
constexpr int MAX_CHUNKS = 128;
constexpr int CB_THREADS = 256;
__global__ __launch_bounds__(CB_THREADS) void attn_combine_kernel(const float* __restrict__ partial,
                                                                  __bf16* __restrict__ out,
                                                                  const int* __restrict__ entries,
                                                                  const int* __restrict__ entry_start, int heads, int hd,
                                                                  int chunks) {
  __shared__ float weight[MAX_CHUNKS];
  __shared__ float wave_best[4], wave_total[4];
  __shared__ f32x4 part_sum[CB_THREADS];
  const int slot = blockIdx.x, h = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t stride = hd + 2;
  const float* src = partial + ((size_t)slot * heads + h) * chunks * stride;
  const int quads = hd / 4;                               // hd is a multiple of 8 and at most 256
  const int parts = CB_THREADS / quads;                   // at least 4
  const int quad = tid % quads, part = tid / quads;
  const bool active = part < parts;
  constexpr int AHEAD = 4;
  const int token = entry_start[entries[slot]];
  f32x4 ahead[AHEAD];
#pragma unroll
  for (int u = 0; u < AHEAD; ++u) {
    const int c = min(part + u * parts, chunks - 1);      // a clamped chunk's value is not used
    ahead[u] = *(const f32x4*)(src + (size_t)c * stride + quad * 4);
  }
  // chunk tid's (max, sum): MAX_CHUNKS <= CB_THREADS
  const float mc = tid < chunks ? src[(size_t)tid * stride + hd] : -INFINITY;
  const float lc = tid < chunks ? src[(size_t)tid * stride + hd + 1] : 0.f;
  float best = wave_max(mc);
  if (lane == 0) wave_best[wave] = best;
  __syncthreads();
  best = fmaxf(fmaxf(wave_best[0], wave_best[1]), fmaxf(wave_best[2], wave_best[3]));
  const float w = mc > -INFINITY ? __expf(mc - best) : 0.f;
  if (tid < chunks) weight[tid] = w;
  const float mine = wave_sum(w * lc);
  if (lane == 0) wave_total[wave] = mine;
  __syncthreads();
  const float inv = 1.f / (((wave_total[0] + wave_total[1]) + wave_total[2]) + wave_total[3]);
  f32x4 acc = {0.f, 0.f, 0.f, 0.f};
  if (active) {
    int c = part;
#pragma unroll
    for (int u = 0; u < AHEAD; ++u, c += parts) {
      if (c >= chunks) break;
      const float wc = weight[c];
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += wc != 0.f ? ahead[u][j] * wc : 0.f;   // an empty chunk holds stale numbers
    }
    for (; c < chunks; c += parts) {
      const float wc = weight[c];
      const f32x4 v = *(const f32x4*)(src + (size_t)c * stride + quad * 4);
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] += wc != 0.f ? v[j] * wc : 0.f;
    }
  }
  part_sum[tid] = acc;
  __syncthreads();
  if (tid < quads) {
    acc = part_sum[tid];
    for (int p = 1; p < parts; ++p) acc += part_sum[p * quads + tid];
    bf16x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) r[j] = (__bf16)(acc[j] * inv);
    *(bf16x4*)(out + (size_t)token * heads * hd + (size_t)h * hd + tid * 4) = r;
  }
}
}  // namespace

extern "C" int vk_attn_bf16_hdp() { return HDP; }

// tiles: pairs (entry, first token of the tile within the entry), 128 tokens per tile; best sorted by the
// number of positions a tile sees, rising (any order gives the same result). split: nonzero asks for workgroups
// of sixteen waves that halve a tile's positions between them, where the kernel in use has that form (few tiles
// of very different lengths); the result is the same up to rounding.
// chunk_tiles > 0 (with the kernel that loads straight into LDS; ignored otherwise): a tile's steps of 64 positions
// are cut into chunks of that many, a workgroup each, of which no tile has more than `max_chunks`; `partial` holds
// num_tiles * heads * max_chunks * 128 * (padded head width + 4) floats.
extern "C" int vk_attn_bf16_prefill(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                                    void* out, const int* tiles, int num_tiles, const int* entry_start,
                                    const int* entry_first_pos, const int* block_table, int table_width,
                                    int block_size, int heads, int kv_heads, int hd, float scale, int window,
                                    int split, float* partial, long long partial_floats, int chunk_tiles,
                                    int max_chunks, void* stream) {
  if (num_tiles <= 0) return 0;
  if (hd <= 0 || hd > HDP || (hd & 7) || block_size <= 0 || (block_size & 7) || heads <= 0 || kv_heads <= 0 ||
      heads % kv_heads || (q_stride & 7) || window < 0)
    return VK_UNSUPPORTED_SIZE;
  constexpr int lds_bytes = (PT_KV * PT_KROW + HDP * PT_VROW) * (int)sizeof(__bf16);
  // page sizes that are powers of two dividing 64 take the kernel with fixed piece addresses
  const bool fast = (block_size & (block_size - 1)) == 0 && block_size <= PT_KV &&
                    (long long)kv_heads * block_size * hd * 2 < (1ll << 32);
  auto kernel = fast ? attn_prefill_kernel<true> : attn_prefill_kernel<false>;
  static bool configured[2] = {false, false};
  if (!configured[fast]) {
    hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return (int)e;
    configured[fast] = true;
  }
  static int cus = 0;  // compute units of the device, for the pairing of long and short tiles
  if (cus == 0) {
    int device = 0, count = 0;
    hipError_t e = hipGetDevice(&device);
    if (e == hipSuccess) e = hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device);
    if (e != hipSuccess) return (int)e;
    cus = count > 0 ? count : 1;
  }
  if ((long long)num_tiles * heads > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
#ifdef VK_PREFILL_DIRECT
  if (fast && hd == HDP && block_size >= 8 && chunk_tiles > 0) {  // the kernel that loads straight into LDS, in chunks
    if (max_chunks <= 0 || !partial || ((uintptr_t)partial & 15) ||
        (long long)num_tiles * heads * max_chunks * PT_TOKENS * PD_PARTIAL_ROW > partial_floats)
      return VK_BAD_ARGUMENT;
    if ((long long)num_tiles * heads * max_chunks > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
    auto chunked = attn_prefill_direct_kernel<false, true>;
    static bool chunked_configured = false;
    if (!chunked_configured) {
      hipError_t e = hipFuncSetAttribute((const void*)chunked, hipFuncAttributeMaxDynamicSharedMemorySize, 2 * PD_STAGE);
      if (e != hipSuccess) return (int)e;
      chunked_configured = true;
    }
    chunked<<<num_tiles * heads * max_chunks, PT_THREADS, 2 * PD_STAGE, (hipStream_t)stream>>>(
        (const __bf16*)q, q_stride, (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, tiles, entry_start,
        entry_first_pos, block_table, table_width, block_size, heads, kv_heads, scale, window, cus, partial,
        chunk_tiles, max_chunks);
    VK_LAUNCH_CHECK();
    attn_prefill_merge_kernel<<<dim3(num_tiles, heads, PT_TOKENS * (HDP / 4) / 256), 256, 0, (hipStream_t)stream>>>(
        partial, (__bf16*)out, tiles, entry_start, entry_first_pos, heads, scale, window, chunk_tiles, max_chunks);
    VK_LAUNCH_CHECK();
    return 0;
  }
  if (fast && hd == HDP && block_size >= 8) {  // the kernel that loads straight into LDS
    const bool halves = split != 0 && PD_CAN_SPLIT;
    auto direct = attn_prefill_direct_kernel<false>;
    if constexpr (PD_CAN_SPLIT) {
      if (halves) direct = attn_prefill_direct_kernel<true>;
    }
    const int direct_lds = (halves ? 4 : 2) * PD_STAGE;
    static bool direct_configured[2] = {false, false};
    if (!direct_configured[halves]) {
      hipError_t e = hipFuncSetAttribute((const void*)direct, hipFuncAttributeMaxDynamicSharedMemorySize, direct_lds);
      if (e != hipSuccess) return (int)e;
      direct_configured[halves] = true;
    }
    direct<<<num_tiles * heads, halves ? 2 * PT_THREADS : PT_THREADS, direct_lds, (hipStream_t)stream>>>(
        (const __bf16*)q, q_stride, (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, tiles, entry_start,
        entry_first_pos, block_table, table_width, block_size, heads, kv_heads, scale, window, cus, nullptr, 0, 1);
    VK_LAUNCH_CHECK();
    return 0;
  }
#endif
  kernel<<<num_tiles * heads, PT_THREADS, lds_bytes, (hipStream_t)stream>>>(
      (const __bf16*)q, q_stride, (const __bf16*)k_cache, (const __bf16*)v_cache, (__bf16*)out, tiles, entry_start,
      entry_first_pos, block_table, table_width, block_size, heads, kv_heads, hd, scale, window, cus);
  VK_LAUNCH_CHECK();
  return 0;
}

// entries: indices of the step's entries that hold exactly one token. partial: at least
// num_entries * heads * chunks * (hd + 2) floats. `chunks` must cover the longest visible range:
// chunks * chunk >= longest position + 1. `join` nonzero: one workgroup of `chunks` waves (at most 8) per entry and
// key head merges its chunks itself and writes `out`; `partial` is not used and may be null.
extern "C" int vk_attn_bf16_decode(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                                   void* out, float* partial, const int* entries, int num_entries,
                                   const int* entry_start, const int* entry_first_pos, const int* block_table,
                                   int table_width, int block_size, int heads, int kv_heads, int hd, float scale,
                                   int window, int chunk, int chunks, int dense, int join, void* stream) {
  if (num_entries <= 0) return 0;
  if (hd <= 0 || hd > HDP || (hd & 7) || block_size <= 0 || (block_size & 7) || heads <= 0 || kv_heads <= 0 ||
      heads % kv_heads || (q_stride & 7) || window < 0 || chunk < 32 || (chunk & 31) || chunks <= 0 ||
      chunks > MAX_CHUNKS)
    return VK_UNSUPPORTED_SIZE;
  if (join && chunks > JOINED_WAVES) return VK_UNSUPPORTED_SIZE;
  if (!join && !partial) return VK_BAD_ARGUMENT;
  const int group = heads / kv_heads, head_blocks = (group + 15) / 16;
  if (kv_heads * head_blocks > 65535 || heads > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  // pages a chunk can touch: chunks start at multiples of `chunk`, which need not be page edges
  const int chunk_pages = chunk % block_size == 0 ? chunk / block_size : chunk / block_size + 2;
  if (join) {
    auto kernel = chunk_pages <= 64 ? attn_decode_kernel<true, true> : attn_decode_kernel<false, true>;
    const int lds_bytes = chunks * (DT * 64 * 16 + 16 * 2 * 4);
    static bool configured[2] = {false, false};
    if (!configured[chunk_pages <= 64]) {
      hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                         JOINED_WAVES * (DT * 64 * 16 + 16 * 2 * 4));
      if (e != hipSuccess) return (int)e;
      configured[chunk_pages <= 64] = true;
    }
    kernel<<<dim3(num_entries, kv_heads * head_blocks), chunks * 64, lds_bytes, s>>>(
        (const __bf16*)q, q_stride, (const __bf16*)k_cache, (const __bf16*)v_cache, nullptr, (__bf16*)out, entries,
        entry_start, entry_first_pos, block_table, table_width, block_size, heads, kv_heads, hd, scale, window, chunk,
        head_blocks, dense);
    VK_LAUNCH_CHECK();
    return 0;
  }
  dim3 grid(num_entries, kv_heads * head_blocks, chunks);
  auto kernel = chunk_pages <= 64 ? attn_decode_kernel<true, false> : attn_decode_kernel<false, false>;
  kernel<<<grid, 64, 0, s>>>((const __bf16*)q, q_stride, (const __bf16*)k_cache, (const __bf16*)v_cache, partial,
                             (__bf16*)out, entries, entry_start, entry_first_pos, block_table, table_width, block_size,
                             heads, kv_heads, hd, scale, window, chunk, head_blocks, dense);
  VK_LAUNCH_CHECK();
  dim3 cgrid(num_entries, heads);
  attn_combine_kernel<<<cgrid, CB_THREADS, 0, s>>>(partial, (__bf16*)out, entries, entry_start, heads, hd, chunks);
  VK_LAUNCH_CHECK();
  return 0;
}
