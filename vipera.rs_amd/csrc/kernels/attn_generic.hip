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
    float scale, int window) {
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
}  // namespace

extern "C" int vk_attn_generic(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                               void* out, int dtype, const int* positions, const int* entry_of_token,
                               const int* block_table, int table_width, int block_size, int num_tokens, int heads,
                               int kv_heads, int hd, float scale, int window, void* stream) {
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
                                                        heads, kv_heads, hd, scale, window);
  else if (dtype == DT_BF16)
    attn_generic_kernel<bf16_t><<<grid, THREADS, 0, s>>>((const bf16_t*)q, q_stride, (const bf16_t*)k_cache,
                                                         (const bf16_t*)v_cache, (bf16_t*)out, positions,
                                                         entry_of_token, block_table, table_width, block_size,
                                                         heads, kv_heads, hd, scale, window);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}
