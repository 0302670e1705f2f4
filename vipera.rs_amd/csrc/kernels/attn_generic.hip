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
    for (int it = 0; it < DEC_WAVE / 4; ++it) {
      const int p = wave_begin + it * 4 + ps;
      const int pc = min(max(p, lo), pos);       // a position outside the range reads one inside it; its score is masked
      const float* row = k_cache + (((size_t)table[pc / block_size] * kv_heads + kvh) * block_size + pc % block_size) * hd;
      float dot[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) dot[h] = 0.f;
#pragma unroll
      for (int i = 0; i < QC; ++i) {
        const int d = c * 4 + 64 * i;
        if (d < hd) {
          const f32x4 k4 = *(const f32x4*)(row + d);
#pragma unroll
          for (int h = 0; h < HB; ++h) {
            dot[h] = fmaf(qr[h][i][0], k4[0], dot[h]);
            dot[h] = fmaf(qr[h][i][1], k4[1], dot[h]);
            dot[h] = fmaf(qr[h][i][2], k4[2], dot[h]);
            dot[h] = fmaf(qr[h][i][3], k4[3], dot[h]);
          }
        }
      }
#pragma unroll
      for (int h = 0; h < HB; ++h) {
#pragma unroll
        for (int off = 1; off < 16; off <<= 1) dot[h] += __shfl_xor(dot[h], off, WAVE);
        if (c == 0) sw[wave][h][it * 4 + ps] = (p >= lo && p <= pos) ? dot[h] * scale : -INFINITY;
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
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p0 = wave_begin + (qs + 4 * j) * 4;             // four positions of one page
      if (p0 > pos || p0 + 3 < lo) continue;
      bool sees[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) sees[e] = p0 + e >= lo && p0 + e <= pos;
      const float* page = v_cache + ((size_t)table[p0 / block_size] * kv_heads + kvh) * hd * block_size + p0 % block_size;
      f32x4 w4[HB];
#pragma unroll
      for (int h = 0; h < HB; ++h) w4[h] = *(const f32x4*)&sw[wave][h][(qs + 4 * j) * 4];
#pragma unroll
      for (int i = 0; i < OD; ++i) {
        const int d = dg + 16 * i;
        if (d < hd) {
          f32x4 v4 = *(const f32x4*)(page + (size_t)d * block_size);
#pragma unroll
          for (int e = 0; e < 4; ++e) v4[e] = sees[e] ? v4[e] : 0.f;
#pragma unroll
          for (int h = 0; h < HB; ++h) {
            o[h][i] = fmaf(w4[h][0], v4[0], o[h][i]);
            o[h][i] = fmaf(w4[h][1], v4[1], o[h][i]);
            o[h][i] = fmaf(w4[h][2], v4[2], o[h][i]);
            o[h][i] = fmaf(w4[h][3], v4[3], o[h][i]);
          }
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
