// Causal grouped-query attention over the paged cache, one workgroup per (token, query head),
// all arithmetic in 32-bit. It serves prompts and decoded tokens alike: a token at position
// `pos` reads the keys at [lo, pos], lo = 0 or pos + 1 - window, from its own request's pages.
// The cache already holds the keys and values of every token of the step.
//
// Formula of the reference (crates/vipera-backend-cpu/src/model.rs:1811-1857): head h uses key
// head h / (heads / kv_heads); score = dot(q, k) * scale with the scale applied after the dot;
// softmax over the visible positions; output = sum of weight * v. The window keeps the last
// `window` positions, the current one included (model.rs:2509). Here the softmax is computed
// online over tiles of 256 keys that start at lo, so the arithmetic of a token depends only on
// its position and the cache contents, not on how the step was cut or batched.
//
// Cache layout: K [page, kv_head, slot, head_dim], V transposed [page, kv_head, head_dim, slot];
// page of position p = table[entry, p / block_size].
#include "common.h"

namespace {
constexpr int THREADS = 256;
constexpr int MAX_HD = 256;

template <typename T>
__global__ __launch_bounds__(THREADS) void attn_generic_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    T* __restrict__ out, const int* __restrict__ positions, const int* __restrict__ entry_of_token,
    const int* __restrict__ block_table, int table_width, int block_size, int heads, int kv_heads, int hd,
    float scale, int window, const int* __restrict__ skip_single_of) {
  // skip_single_of (entry_start, or null): tokens of entries that hold one token are left to the decode kernel
  if (skip_single_of) {
    const int e = entry_of_token[blockIdx.x];
    if (skip_single_of[e + 1] - skip_single_of[e] == 1) return;
  }
  __shared__ float q_s[MAX_HD];
  __shared__ float p_s[THREADS];
  __shared__ int page_s[THREADS];
  __shared__ float red[16];
  __shared__ float part_s[THREADS];

  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (heads / kv_heads);
  const int pos = positions[t];
  const int hi = pos + 1;
  const int lo = (window > 0 && hi > window) ? hi - window : 0;
  const int* table = block_table + (size_t)entry_of_token[t] * table_width;

  for (int d = tid; d < hd; d += THREADS) q_s[d] = to_float<T>(q[(size_t)t * q_stride + (size_t)h * hd + d]);

  // value phase mapping: thread -> (part, d); part p takes keys j with j % parts == p
  const int parts = THREADS / hd > 0 ? THREADS / hd : 1;
  const int vd = tid % hd, vpart = tid / hd;
  const bool v_active = vpart < parts;
  float acc = 0.f, m = -INFINITY, l = 0.f;
  __syncthreads();

  for (int base = lo; base < hi; base += THREADS) {
    const int p = base + tid;
    float s = -INFINITY;
    int page = -1;
    if (p < hi) {
      page = table[p / block_size];
      const T* k_row = k_cache + (((size_t)page * kv_heads + kvh) * block_size + (p % block_size)) * hd;
      float dot = 0.f;
      for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], to_float<T>(k_row[d]), dot);
      s = dot * scale;
    }
    const float tile_max = block_max(s, red);
    const float m_new = fmaxf(m, tile_max);
    const float w = (p < hi) ? expf(s - m_new) : 0.f;
    const float tile_sum = block_sum(w, red);
    const float rescale = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * rescale + tile_sum;
    m = m_new;
    p_s[tid] = w;
    page_s[tid] = page;
    __syncthreads();
    if (v_active) {
      acc *= rescale;
      const int count = min(THREADS, hi - base);
      for (int j = vpart; j < count; j += parts) {
        const int pj = base + j;
        const T* v_at = v_cache + (((size_t)page_s[j] * kv_heads + kvh) * hd + vd) * block_size + (pj % block_size);
        acc = fmaf(p_s[j], to_float<T>(*v_at), acc);
      }
    }
    __syncthreads();
  }
  // sum the parts in a fixed order
  part_s[tid] = v_active ? acc : 0.f;
  __syncthreads();
  if (tid < hd) {
    float total = 0.f;
    for (int pidx = 0; pidx < parts; ++pidx) total += part_s[pidx * hd + tid];
    out[(size_t)t * heads * hd + (size_t)h * hd + tid] = from_float<T>(total / l);
  }
}

// ---------------------------------------------------------------------------------------------
// Decoding in 32-bit: entries that hold one token. The kernel above gives such a token one workgroup per query
// head, which walks all of its positions alone and reads every key and value once per query head; with a few
// requests of thousands of positions that is a handful of workgroups reading the cache seven times over. Here a
// workgroup owns (entry, key head, chunk of 256 positions) and up to HB query heads of the key head share every
// read; the chunks' (max, sum, weighted sum) are merged by a second kernel in ascending order, as the
// reference's split kernels do (crates/vipera-backend-gpu/src/layer.cu:307-467). A wave owns 64 positions:
//   scores   16 lanes per position, each 4 dims of every 64 (a wave's load is four whole K rows, which lie
//            one after another in a page), the dot products summed over the 16 lanes in a fixed tree;
//   softmax  a lane per position: maximum, exp (library grade), sum over the wave in a fixed tree;
//   output   a lane owns dims dg, dg + 16, ... and every fourth quad of positions (V pages are stored
//            transposed, so four positions of a dim are 16 bytes); a position that the token does not see
//            counts as zero whatever its slot holds, not as its weight of zero times that.
// Which positions a chunk and a wave hold depends on the position alone, so a token's arithmetic does not
// depend on its company. Needs a head width that is a multiple of 4 and pages of a multiple of 4 positions.
constexpr int DEC_CHUNK = 256, DEC_WAVE = 64;

template <int HB, int QC>   // HB query heads together; QC chunks of 64 dims cover the head width
__global__ __launch_bounds__(256) void attn_decode_f32_kernel(
    const float* __restrict__ q, long long q_stride, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, float* __restrict__ partial, const int* __restrict__ entries,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos,
    const int* __restrict__ block_table, int table_width, int block_size, int heads, int kv_heads, int hd,
    float scale, int window, int head_blocks) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  __shared__ float sw[4][HB][DEC_WAVE];                 // a wave's scores, then its weights
  __shared__ float merge_o[4][HB][MAX_HD];              // the waves' weighted sums
  __shared__ float merge_ml[4][HB][2];                  // and their (max, sum)
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int slot_index = blockIdx.x, entry = entries[slot_index];
  const int kvh = blockIdx.y / head_blocks, hb = blockIdx.y % head_blocks;
  const int group = heads / kv_heads;
  const int token = entry_start[entry], pos = entry_first_pos[entry];
  const int lo = (window > 0 && pos + 1 > window) ? pos + 1 - window : 0;
  const int chunk_begin = blockIdx.z * DEC_CHUNK;
  const int first_head = kvh * group + hb * HB;                       // of this block of heads
  const int block_heads = min(HB, group - hb * HB);
  const size_t stride = hd + 2;
  float* dst = partial + (((size_t)slot_index * heads + first_head) * gridDim.z + blockIdx.z) * stride;
  const size_t head_stride = (size_t)gridDim.z * stride;
  if (chunk_begin > pos || chunk_begin + DEC_CHUNK <= lo) {           // nothing of this chunk is visible
    if ((int)threadIdx.x < block_heads) {
      dst[threadIdx.x * head_stride + hd] = -INFINITY;
      dst[threadIdx.x * head_stride + hd + 1] = 0.f;
    }
    return;
  }
  const int* table = block_table + (size_t)entry * table_width;
  const int wave_begin = chunk_begin + wave * DEC_WAVE;
  const bool wave_sees = wave_begin <= pos && wave_begin + DEC_WAVE > lo;

  // ---- scores
  const int ps = lane >> 4, c = lane & 15;
  f32x4 qr[HB][QC];
#pragma unroll
  for (int h = 0; h < HB; ++h)
#pragma unroll
    for (int i = 0; i < QC; ++i) {
      const int d = c * 4 + 64 * i;
      qr[h][i] = (h < block_heads && d < hd) ? *(const f32x4*)(q + (size_t)token * q_stride + (size_t)(first_head + h) * hd + d)
                                             : f32x4{0.f, 0.f, 0.f, 0.f};
    }
  if (wave_sees) {
    // Eight steps of four positions at a time: their page ids are requested together, then their K rows, and only
    // then is anything multiplied. A step at a time (look up the page, wait, fetch the row, wait, multiply) made
    // the kernel sixteen pairs of round trips long: 96 us a layer for 134 MB at the 7B shape. No load sits behind
    // a condition: a dim past the head width reads the last four dims again (its q is zero).
    constexpr int AHEAD = 8;
    for (int it0 = 0; it0 < DEC_WAVE / 4; it0 += AHEAD) {
      int at[AHEAD], page[AHEAD];
#pragma unroll
      for (int b = 0; b < AHEAD; ++b) {
        const int p = wave_begin + (it0 + b) * 4 + ps;
        at[b] = min(max(p, lo), pos);   // a position outside the range reads one inside it; its score is masked
        page[b] = table[at[b] / block_size];
      }
      f32x4 k4[AHEAD][QC];
#pragma unroll
      for (int b = 0; b < AHEAD; ++b) {
        const float* row = k_cache + (((size_t)page[b] * kv_heads + kvh) * block_size + at[b] % block_size) * hd;
#pragma unroll
        for (int i = 0; i < QC; ++i) k4[b][i] = *(const f32x4*)(row + min(c * 4 + 64 * i, hd - 4));
      }
#pragma unroll
      for (int b = 0; b < AHEAD; ++b) {
        const int p = wave_begin + (it0 + b) * 4 + ps;
        float dot[HB];
#pragma unroll
        for (int h = 0; h < HB; ++h) dot[h] = 0.f;
#pragma unroll
        for (int i = 0; i < QC; ++i)
#pragma unroll
          for (int h = 0; h < HB; ++h) {
            dot[h] = fmaf(qr[h][i][0], k4[b][i][0], dot[h]);
            dot[h] = fmaf(qr[h][i][1], k4[b][i][1], dot[h]);
            dot[h] = fmaf(qr[h][i][2], k4[b][i][2], dot[h]);
            dot[h] = fmaf(qr[h][i][3], k4[b][i][3], dot[h]);
          }
#pragma unroll
        for (int h = 0; h < HB; ++h) {
#pragma unroll
          for (int off = 1; off < 16; off <<= 1) dot[h] += __shfl_xor(dot[h], off, WAVE);
          if (c == 0) sw[wave][h][(it0 + b) * 4 + ps] = (p >= lo && p <= pos) ? dot[h] * scale : -INFINITY;
        }
      }
    }
  }
  __syncthreads();
  // ---- softmax over the wave's 64 positions, a lane per position
  float m[HB], l[HB];
#pragma unroll
  for (int h = 0; h < HB; ++h) {
    const float sc = wave_sees ? sw[wave][h][lane] : -INFINITY;
    m[h] = wave_max(sc);
    const float w = m[h] > -INFINITY ? expf(sc - m[h]) : 0.f;
    l[h] = wave_sum(w);
    sw[wave][h][lane] = w;
  }
  __syncthreads();
  // ---- output: lane (dg, qs) owns dims dg + 16 i and the quads of positions qs, qs + 4, qs + 8, qs + 12
  constexpr int OD = QC * 4;                  // 16-dim steps that cover the head width
  const int dg = lane >> 2, qs = lane & 3;
  float o[HB][OD];
#pragma unroll
  for (int h = 0; h < HB; ++h)
#pragma unroll
    for (int i = 0; i < OD; ++i) o[h][i] = 0.f;
  if (wave_sees) {
    // the four quads' pages first, then their values, no load behind a condition: a quad of which the token sees
    // nothing reads the quad of its own position instead (whose page is held) and counts as zeros
    const float* quad[4];
    bool sees[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p0 = wave_begin + (qs + 4 * j) * 4;             // four positions of one page
      const bool any = p0 <= pos && p0 + 3 >= lo;
      const int from = any ? p0 : (pos & ~3);
#pragma unroll
      for (int e = 0; e < 4; ++e) sees[j][e] = any && p0 + e >= lo && p0 + e <= pos;
      quad[j] = v_cache + ((size_t)table[from / block_size] * kv_heads + kvh) * hd * block_size + from % block_size;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f32x4 v4[OD];
#pragma unroll
      for (int i = 0; i < OD; ++i) v4[i] = *(const f32x4*)(quad[j] + (size_t)min(dg + 16 * i, hd - 1) * block_size);
      f32x4 w4[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) w4[h] = *(const f32x4*)&sw[wave][h][(qs + 4 * j) * 4];
#pragma unroll
      for (int i = 0; i < OD; ++i) {
#pragma unroll
        for (int e = 0; e < 4; ++e) v4[i][e] = sees[j][e] ? v4[i][e] : 0.f;
#pragma unroll
        for (int h = 0; h < HB; ++h) {   // a dim past the head width adds into a sum that is never stored
          o[h][i] = fmaf(w4[h][0], v4[i][0], o[h][i]);
          o[h][i] = fmaf(w4[h][1], v4[i][1], o[h][i]);
          o[h][i] = fmaf(w4[h][2], v4[i][2], o[h][i]);
          o[h][i] = fmaf(w4[h][3], v4[i][3], o[h][i]);
        }
      }
    }
  }
#pragma unroll
  for (int h = 0; h < HB; ++h) {
#pragma unroll
    for (int i = 0; i < OD; ++i) {
      float v = o[h][i];
      v += __shfl_xor(v, 1, WAVE);
      v += __shfl_xor(v, 2, WAVE);
      if (qs == 0 && dg + 16 * i < hd) merge_o[wave][h][dg + 16 * i] = v;
    }
    if (lane == 0) {
      merge_ml[wave][h][0] = m[h];
      merge_ml[wave][h][1] = l[h];
    }
  }
  __syncthreads();
  // ---- the four waves' results merged in ascending order
  for (int at = threadIdx.x; at < block_heads * hd; at += 256) {
    const int h = at / hd, d = at % hd;
    float best = -INFINITY;
#pragma unroll
    for (int w = 0; w < 4; ++w) best = fmaxf(best, merge_ml[w][h][0]);
    float total = 0.f, sum = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float mw = merge_ml[w][h][0];
      if (mw > -INFINITY) {
        const float factor = expf(mw - best);
        total = fmaf(merge_o[w][h][d], factor, total);
        sum = fmaf(merge_ml[w][h][1], factor, sum);
      }
    }
    dst[h * head_stride + d] = total;
    if (d == 0) {
      dst[h * head_stride + hd] = best;
      dst[h * head_stride + hd + 1] = sum;
    }
  }
}

// out = sum_c acc_c e^(m_c - M) / sum_c l_c e^(m_c - M) over the chunks in ascending order, M their largest maximum.
template <typename T>
__global__ __launch_bounds__(64) void attn_combine_f32_kernel(const float* __restrict__ partial, T* __restrict__ out,
                                                              const int* __restrict__ entries,
                                                              const int* __restrict__ entry_start, int heads, int hd,
                                                              int chunks) {
  const int slot_index = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const size_t stride = hd + 2;
  const float* src = partial + ((size_t)slot_index * heads + h) * chunks * stride;
  float best = -INFINITY;
  for (int ch = lane; ch < chunks; ch += 64) best = fmaxf(best, src[(size_t)ch * stride + hd]);
  best = wave_max(best);
  const int token = entry_start[entries[slot_index]];
  for (int d = lane; d < hd; d += 64) {
    float total = 0.f, sum = 0.f;
    for (int ch = 0; ch < chunks; ++ch) {
      const float mc = src[(size_t)ch * stride + hd];
      if (mc > -INFINITY) {      // an empty chunk's sums hold nothing
        const float factor = expf(mc - best);
        total = fmaf(src[(size_t)ch * stride + d], factor, total);
        sum = fmaf(src[(size_t)ch * stride + hd + 1], factor, sum);
      }
    }
    out[(size_t)token * heads * hd + (size_t)h * hd + d] = from_float<T>(total / sum);
  }
}

// ---------------------------------------------------------------------------------------------
// Prompt portions in 32-bit. The general kernel gives every (token, query head) a workgroup that walks all of the
// token's positions alone: 2,048 tokens x 28 heads read the cache 58 GB over per layer. Here a workgroup owns 64
// consecutive tokens of one entry and one query head and walks the positions in tiles of 64 that begin at
// multiples of 64 (so which positions share a tile, and with it a token's arithmetic, depends on the position alone,
// not on how the prompt was cut): the K tile and the V^T tile go into LDS as they lie in the pages (rows padded by 16
// bytes, so that sixteen lanes reading sixteen consecutive rows spread over the banks), slots past the last
// position of the tile's tokens as zeros (a weight of zero times whatever a free slot holds must stay zero), and so
// are positions before the first one that the tile's first token sees: a window has passed them, and their page
// may have been given back (its id in the table is then -1 and must not be followed).
//   scores   thread (ty, tx) of 16 x 16 owns tokens 4 ty .. 4 ty + 3 and positions tx, tx + 16, tx + 32, tx + 48: a
//            dot product is an FMA chain over the head width in ascending order;
//   softmax  online over the tiles (crates/vipera-backend-cpu/src/model.rs:1840-1857 is the plain form): a row's
//            maximum and sum over the sixteen lanes that share it in a fixed tree, library-grade exp;
//   output   the weights go through LDS; thread (ty, tx) owns the same four tokens and dims tx, tx + 16, ...: an
//            FMA chain over the tile's positions in ascending order.
// Head widths that are multiples of 16 up to 128 (the tiles of a wider head do not fit a CU's LDS) and pages of a
// multiple of 4 positions; anything else stays with the general kernel.
constexpr int PF_TILE = 64;
template <int DPT>   // the head width is 16 * DPT
__global__ __launch_bounds__(256) void attn_prefill_f32_kernel(
    const float* __restrict__ q, long long q_stride, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, float* __restrict__ out, const int* __restrict__ tiles,
    const int* __restrict__ entry_start, const int* __restrict__ entry_first_pos, const int* __restrict__ block_table,
    int table_width, int block_size, int heads, int kv_heads, float scale, int window, int tile_tokens) {
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  constexpr int HD = 16 * DPT, QROW = HD + 4, VROW = PF_TILE + 4;
  extern __shared__ __attribute__((aligned(16))) float pf_lds[];
  float* q_s = pf_lds;                     // [64][QROW]
  float* k_s = q_s + PF_TILE * QROW;       // [64][QROW]
  float* v_s = k_s + PF_TILE * QROW;       // [HD][VROW], transposed as in the pages
  float* p_s = v_s + HD * VROW;            // [64][VROW]
  const int parts = tile_tokens / PF_TILE;                 // workgroups per tile of the step's list
  // the list comes with the tiles that see most positions last; workgroups start in the order of their index, and the
  // long ones should start first, so that the short ones fill the gaps at the end
  const int index = gridDim.x - 1 - blockIdx.x;
  const int tile = index / parts, part = index % parts, h = blockIdx.y;
  const int entry = tiles[2 * tile], offset = tiles[2 * tile + 1] + part * PF_TILE;
  const int count = entry_start[entry + 1] - entry_start[entry];
  if (offset >= count) return;
  const int rows = min(PF_TILE, count - offset);
  const int tok0 = entry_start[entry] + offset, pos0 = entry_first_pos[entry] + offset;
  const int last_pos = pos0 + rows - 1;
  const int kvh = h / (heads / kv_heads);
  const int* table = block_table + (size_t)entry * table_width;
  const int tid = threadIdx.x, ty = tid >> 4, tx = tid & 15;

  for (int i = tid; i < PF_TILE * (HD / 4); i += 256) {
    const int r = i / (HD / 4), c = (i % (HD / 4)) * 4;
    f32x4 v = {0.f, 0.f, 0.f, 0.f};
    if (r < rows) v = *(const f32x4*)(q + (size_t)(tok0 + r) * q_stride + (size_t)h * HD + c);
    *(f32x4*)(q_s + r * QROW + c) = v;
  }
  float m[4], l[4], o[4][DPT];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    m[i] = -INFINITY;
    l[i] = 0.f;
#pragma unroll
    for (int j = 0; j < DPT; ++j) o[i][j] = 0.f;
  }
  const int lowest = (window > 0 && pos0 + 1 > window) ? pos0 + 1 - window : 0;   // the first token's first position
  for (int kv0 = lowest / PF_TILE * PF_TILE; kv0 <= last_pos; kv0 += PF_TILE) {
    __syncthreads();   // the tile before has been read
    for (int i = tid; i < PF_TILE * (HD / 4); i += 256) {
      const int r = i / (HD / 4), c = (i % (HD / 4)) * 4, p = kv0 + r;
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (p >= lowest && p <= last_pos)   // below `lowest` the window has passed: the page may have been given back
        v = *(const f32x4*)(k_cache + (((size_t)table[p / block_size] * kv_heads + kvh) * block_size + p % block_size) * HD + c);
      *(f32x4*)(k_s + r * QROW + c) = v;
    }
    for (int i = tid; i < HD * (PF_TILE / 4); i += 256) {
      const int d = i / (PF_TILE / 4), c = (i % (PF_TILE / 4)) * 4, p = kv0 + c;   // four positions of one page
      f32x4 v = {0.f, 0.f, 0.f, 0.f};
      if (p + 3 >= lowest && p <= last_pos) {   // the four share a page, which is held if any of them is visible
        v = *(const f32x4*)(v_cache + (((size_t)table[p / block_size] * kv_heads + kvh) * HD + d) * block_size + p % block_size);
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (p + e < lowest || p + e > last_pos) v[e] = 0.f;
      }
      *(f32x4*)(v_s + d * VROW + c) = v;
    }
    __syncthreads();
    float s[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) s[i][j] = 0.f;
    auto score_step = [&](int c) {
      f32x4 qv[4], kv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) qv[i] = *(const f32x4*)(q_s + (4 * ty + i) * QROW + c);
#pragma unroll
      for (int j = 0; j < 4; ++j) kv[j] = *(const f32x4*)(k_s + (tx + 16 * j) * QROW + c);
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          s[i][j] = fmaf(qv[i][0], kv[j][0], s[i][j]);
          s[i][j] = fmaf(qv[i][1], kv[j][1], s[i][j]);
          s[i][j] = fmaf(qv[i][2], kv[j][2], s[i][j]);
          s[i][j] = fmaf(qv[i][3], kv[j][3], s[i][j]);
        }
    };
    // A head of up to 64 dims is few enough steps for the compiler to unroll them all and hoist every load, which
    // spills 96 registers at a width of 64: two steps at a time there (2,048 tokens of 14 heads 902 to 372 us; a
    // width of 32 191 to 202). Wider heads keep the compiler's own choice (limited to two, a width of 128 ran 15 %
    // slower).
    if constexpr (DPT <= 4) {
#pragma unroll 2
      for (int c = 0; c < HD; c += 4) score_step(c);
    } else {
      for (int c = 0; c < HD; c += 4) score_step(c);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int qpos = pos0 + 4 * ty + i;
      const int first = (window > 0 && qpos + 1 > window) ? qpos + 1 - window : 0;
      float best = -INFINITY;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int p = kv0 + tx + 16 * j;
        const bool sees = 4 * ty + i < rows && p <= qpos && p >= first;
        s[i][j] = sees ? s[i][j] * scale : -INFINITY;
        best = fmaxf(best, s[i][j]);
      }
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) best = fmaxf(best, __shfl_xor(best, off));
      const float m_new = fmaxf(m[i], best);
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float w = s[i][j] > -INFINITY ? expf(s[i][j] - m_new) : 0.f;
        p_s[(4 * ty + i) * VROW + tx + 16 * j] = w;
        sum += w;
      }
#pragma unroll
      for (int off = 1; off < 16; off <<= 1) sum += __shfl_xor(sum, off);
      const float rescale = m[i] > -INFINITY ? expf(m[i] - m_new) : 0.f;   // nothing seen so far: the sums are zero
      l[i] = l[i] * rescale + sum;
      m[i] = m_new;
#pragma unroll
      for (int j = 0; j < DPT; ++j) o[i][j] *= rescale;
    }
    __syncthreads();
    auto output_step = [&](int c) {
      f32x4 pv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) pv[i] = *(const f32x4*)(p_s + (4 * ty + i) * VROW + c);
#pragma unroll
      for (int j = 0; j < DPT; ++j) {
        const f32x4 vv = *(const f32x4*)(v_s + (tx + 16 * j) * VROW + c);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          o[i][j] = fmaf(pv[i][0], vv[0], o[i][j]);
          o[i][j] = fmaf(pv[i][1], vv[1], o[i][j]);
          o[i][j] = fmaf(pv[i][2], vv[2], o[i][j]);
          o[i][j] = fmaf(pv[i][3], vv[3], o[i][j]);
        }
      }
    };
    if constexpr (DPT <= 4) {
#pragma unroll 2
      for (int c = 0; c < PF_TILE; c += 4) output_step(c);
    } else {
      for (int c = 0; c < PF_TILE; c += 4) output_step(c);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if (4 * ty + i >= rows) continue;
    float* dst = out + (size_t)(tok0 + 4 * ty + i) * heads * HD + (size_t)h * HD;
#pragma unroll
    for (int j = 0; j < DPT; ++j) dst[tx + 16 * j] = o[i][j] / l[i];
  }
}

template <int DPT>
int launch_prefill_f32(dim3 grid, hipStream_t s, const float* q, long long q_stride, const float* k_cache,
                       const float* v_cache, float* out, const int* tiles, const int* entry_start,
                       const int* entry_first_pos, const int* block_table, int table_width, int block_size, int heads,
                       int kv_heads, float scale, int window, int tile_tokens) {
  constexpr int HD = 16 * DPT;
  constexpr int lds_bytes = (2 * PF_TILE * (HD + 4) + HD * (PF_TILE + 4) + PF_TILE * (PF_TILE + 4)) * 4;
  static_assert(lds_bytes <= 160 * 1024, "a CU has 160 KB of LDS");
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)attn_prefill_f32_kernel<DPT>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, lds_bytes);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  attn_prefill_f32_kernel<DPT><<<grid, 256, lds_bytes, s>>>(q, q_stride, k_cache, v_cache, out, tiles, entry_start,
                                                            entry_first_pos, block_table, table_width, block_size,
                                                            heads, kv_heads, scale, window, tile_tokens);
  return 0;
}

template <int HB, int QC>
void launch_decode_f32(dim3 grid, hipStream_t s, const float* q, long long q_stride, const float* k_cache,
                       const float* v_cache, float* partial, const int* entries, const int* entry_start,
                       const int* entry_first_pos, const int* block_table, int table_width, int block_size, int heads,
                       int kv_heads, int hd, float scale, int window, int head_blocks) {
  attn_decode_f32_kernel<HB, QC><<<grid, 256, 0, s>>>(q, q_stride, k_cache, v_cache, partial, entries, entry_start,
                                                      entry_first_pos, block_table, table_width, block_size, heads,
                                                      kv_heads, hd, scale, window, head_blocks);
}
}  // namespace

extern "C" int vk_attn_generic(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                               void* out, int dtype, const int* positions, const int* entry_of_token,
                               const int* block_table, int table_width, int block_size, int num_tokens, int heads,
                               int kv_heads, int hd, float scale, int window, const int* skip_single_of,
                               void* stream) {
  if (num_tokens <= 0) return 0;
  if (hd <= 0 || hd > MAX_HD) return VK_UNSUPPORTED_SIZE;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || heads > 65535 || block_size <= 0 || table_width <= 0 ||
      window < 0)
    return VK_BAD_ARGUMENT;
  dim3 grid(num_tokens, heads);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32)
    attn_generic_kernel<float><<<grid, THREADS, 0, s>>>((const float*)q, q_stride, (const float*)k_cache,
                                                        (const float*)v_cache, (float*)out, positions,
                                                        entry_of_token, block_table, table_width, block_size,
                                                        heads, kv_heads, hd, scale, window, skip_single_of);
  else if (dtype == DT_BF16)
    attn_generic_kernel<bf16_t><<<grid, THREADS, 0, s>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
                                                         (const bf16_t*)v_cache, (bf16_t*)out, positions,
                                                         entry_of_token, block_table, table_width, block_size,
                                                         heads, kv_heads, hd, scale, window, skip_single_of);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}


// Positions per chunk of vk_attn_decode_f32: `chunks` must cover the longest visible range.
extern "C" int vk_attn_decode_f32_chunk() { return DEC_CHUNK; }

// Attention of the single-token entries listed in `entries` in 32-bit: float q, cache and out. partial: at least
// num_entries * heads * chunks * (hd + 2) floats; chunks * 256 >= longest position + 1.
extern "C" int vk_attn_decode_f32(const float* q, long long q_stride, const float* k_cache, const float* v_cache,
                                  float* out, float* partial, const int* entries, int num_entries,
                                  const int* entry_start, const int* entry_first_pos, const int* block_table,
                                  int table_width, int block_size, int heads, int kv_heads, int hd, float scale,
                                  int window, int chunks, void* stream) {
  if (num_entries <= 0) return 0;
  if (hd <= 0 || hd > MAX_HD || (hd & 3) || block_size <= 0 || (block_size & 3) || (q_stride & 3)) return VK_UNSUPPORTED_SIZE;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || table_width <= 0 || window < 0 || chunks <= 0 ||
      chunks > 65535)
    return VK_BAD_ARGUMENT;
  if (((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15)) return VK_BAD_ARGUMENT;
  const int group = heads / kv_heads;
  // heads that share the reads: as many as the registers hold beside hd / 16 sums each
  const int qc = (hd + 63) / 64;
  const int most = qc <= 2 ? 8 : 4;
  int hb = 1;
  while (hb < group && hb < most) hb *= 2;
  const int head_blocks = (group + hb - 1) / hb;
  if (kv_heads * head_blocks > 65535 || heads > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(num_entries, kv_heads * head_blocks, chunks);
#define VK_DEC(HBV, QCV)                                                                                          \
  launch_decode_f32<HBV, QCV>(grid, s, q, q_stride, k_cache, v_cache, partial, entries, entry_start, entry_first_pos, \
                              block_table, table_width, block_size, heads, kv_heads, hd, scale, window, head_blocks)
  if (qc == 1) {
    switch (hb) { case 1: VK_DEC(1, 1); break; case 2: VK_DEC(2, 1); break; case 4: VK_DEC(4, 1); break; default: VK_DEC(8, 1); }
  } else if (qc == 2) {
    switch (hb) { case 1: VK_DEC(1, 2); break; case 2: VK_DEC(2, 2); break; case 4: VK_DEC(4, 2); break; default: VK_DEC(8, 2); }
  } else {
    switch (hb) { case 1: VK_DEC(1, 4); break; case 2: VK_DEC(2, 4); break; default: VK_DEC(4, 4); }
  }
#undef VK_DEC
  VK_LAUNCH_CHECK();
  attn_combine_f32_kernel<float><<<dim3(num_entries, heads), 64, 0, s>>>(partial, out, entries, entry_start, heads, hd, chunks);
  VK_LAUNCH_CHECK();
  return 0;
}

// Attention of the step's prompt portions in 32-bit: float q, cache and out. tiles: pairs (entry, first token of the
// tile within the entry), `tile_tokens` tokens a tile (a multiple of 64), as vk_attn_bf16_prefill takes them. Head
// widths that are multiples of 16 up to 128, pages of a multiple of 4 positions.
extern "C" int vk_attn_prefill_f32(const float* q, long long q_stride, const float* k_cache, const float* v_cache,
                                   float* out, const int* tiles, int num_tiles, int tile_tokens, const int* entry_start,
                                   const int* entry_first_pos, const int* block_table, int table_width, int block_size,
                                   int heads, int kv_heads, int hd, float scale, int window, void* stream) {
  if (num_tiles <= 0) return 0;
  if (hd <= 0 || hd > 128 || (hd & 15) || block_size <= 0 || (block_size & 3) || (q_stride & 3)) return VK_UNSUPPORTED_SIZE;
  if (heads <= 0 || kv_heads <= 0 || heads % kv_heads != 0 || heads > 65535 || table_width <= 0 || window < 0 ||
      tile_tokens <= 0 || tile_tokens % PF_TILE)
    return VK_BAD_ARGUMENT;
  if (((uintptr_t)q & 15) || ((uintptr_t)k_cache & 15) || ((uintptr_t)v_cache & 15)) return VK_BAD_ARGUMENT;
  const long long groups = (long long)num_tiles * (tile_tokens / PF_TILE);
  if (groups > 0x7fffffffLL) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  dim3 grid((unsigned)groups, heads);
  int status = 0;
#define VK_PF(DPTV)                                                                                                  \
  case DPTV:                                                                                                         \
    status = launch_prefill_f32<DPTV>(grid, s, q, q_stride, k_cache, v_cache, out, tiles, entry_start, entry_first_pos, \
                                      block_table, table_width, block_size, heads, kv_heads, scale, window, tile_tokens); \
    break;
  switch (hd / 16) { VK_PF(1) VK_PF(2) VK_PF(3) VK_PF(4) VK_PF(5) VK_PF(6) VK_PF(7) VK_PF(8) }
#undef VK_PF
  if (status != 0) return status;
  VK_LAUNCH_CHECK();
  return 0;
}
