// Row-wise and element-wise kernels: embedding gather, RMSNorm, rotary + cache write,
// gated activation, a counter-based normal fill for random weights, and the fetch of a step's metadata from pinned host memory.
//
// Formulas as the reference computes them:
//   embedding   x = table[token, :]                                  crates/vipera-backend-cpu/src/model.rs:607-616
//   RMSNorm     inv = 1/sqrt(mean(x^2) + eps); out = (x*inv)*w       model.rs:4282-4288
//   rotary      pairs (i, i + half): lo*c - hi*s, lo*s + hi*c        model.rs:4225-4251
//   cache write K (after rotation) and V at table[pos / bs], pos % bs model.rs:1495-1542
//   SwiGLU      up * gate / (1 + exp(-gate))                          model.rs:4368-4374
#include "common.h"

// ---------------------------------------------------------------------------------------------
// A step's metadata (tokens, positions, block tables: tens of KB of 32-bit words) fetched by a kernel straight
// from pinned host memory instead of by a copy command: past a few KB the runtime hands a host-to-device copy to
// the copy engine, and the hand-over between the compute queue and that engine left the GPU idle for about 250 us
// before every decode step of 64 requests (3.5 % of the step). `host` must be pinned memory that the device can
// address (the launcher asks the runtime for its device address and refuses anything else, so the kernel is never
// given a pointer it cannot read).
__global__ void fetch_words_kernel(const int* __restrict__ host, int* __restrict__ out, long long count) {
  const long long i = ((long long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (i + 3 < count) {
    *(int4*)(out + i) = *(const int4*)(host + i);
  } else {
    for (long long j = i; j < count; ++j) out[j] = host[j];
  }
}

extern "C" int vk_fetch_words(const void* pinned_host, void* out, long long count, void* stream) {
  if (count <= 0) return 0;
  if (((uintptr_t)pinned_host & 15) || ((uintptr_t)out & 15) || count > (1ll << 31)) return VK_BAD_ARGUMENT;
  void* device_view = nullptr;
  if (hipHostGetDevicePointer(&device_view, const_cast<void*>(pinned_host), 0) != hipSuccess || device_view == nullptr) {
    (void)hipGetLastError();  // not pinned, or not mapped for this device: the caller copies another way
    return VK_UNSUPPORTED_SIZE;
  }
  const long long threads = (count + 3) / 4;
  fetch_words_kernel<<<(unsigned)((threads + 255) / 256), 256, 0, (hipStream_t)stream>>>((const int*)device_view, (int*)out,
                                                                                         count);
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// `source` (may be null): where source[t] >= 0 the token is not tokens[t] but sampled[source[t]], an id
// that an earlier kernel of the stream left on the device (the previous step's sampler), so that a
// step can be launched before its input token has reached the host. An id outside the table reads row 0
// (the sampler leaves -1 where a row of logits held no finite value; the host fails that request).
template <typename TW>
__global__ void embed_gather_kernel(const TW* __restrict__ table, const int* __restrict__ tokens,
                                    const int* __restrict__ source, const int* __restrict__ sampled,
                                    float* __restrict__ out, int width, int vocab) {
  const int t = blockIdx.x;
  int token = tokens[t];
  if (source != nullptr && source[t] >= 0) token = sampled[source[t]];
  if (token < 0 || token >= vocab) token = 0;
  const TW* row = table + (size_t)token * width;
  float* dst = out + (size_t)t * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = to_float<TW>(row[i]);
}

extern "C" int vk_embed_gather(const void* table, int table_dtype, const int* tokens, const int* source,
                               const int* sampled, float* out, int num_tokens, int width, int vocab, void* stream) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || vocab <= 0 || (source != nullptr && sampled == nullptr)) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (table_dtype == DT_F32)
    embed_gather_kernel<float><<<num_tokens, 256, 0, s>>>((const float*)table, tokens, source, sampled, out, width,
                                                          vocab);
  else if (table_dtype == DT_BF16)
    embed_gather_kernel<bf16_t><<<num_tokens, 256, 0, s>>>((const bf16_t*)table, tokens, source, sampled, out, width,
                                                           vocab);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// One block per output row. `rows` (may be null) picks the input row of each output row.
// The row is read once into registers (four floats at a time when the width allows) and the sum of
// squares is reduced in a fixed order.
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <typename TO>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ weight,
                                                      const int* __restrict__ rows, TO* __restrict__ out, int width,
                                                      float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const float* src = x + (size_t)(rows ? rows[r] : r) * width;
  TO* dst = out + (size_t)r * width;
  constexpr int MAXV = 8;  // up to 8 * 4 * 256 = 8192 columns stay in registers
  if ((width & 3) == 0 && width <= MAXV * 4 * 256) {
    // the weights are requested together with the row, not after the sum: a row of a few tokens is all latency,
    // and a second round trip to memory behind the barrier would be a third of it
    f32x4_t v[MAXV], w[MAXV];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int c = (threadIdx.x + 256 * i) * 4;
      if (c < width) {
        v[i] = *(const f32x4_t*)(src + c);
        w[i] = *(const f32x4_t*)(weight + c);
      }
    }
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int c = (threadIdx.x + 256 * i) * 4;
      if (c < width) sum += v[i][0] * v[i][0] + v[i][1] * v[i][1] + v[i][2] * v[i][2] + v[i][3] * v[i][3];
    }
    sum = block_sum(sum, scratch);
    const float inv = 1.0f / sqrtf(sum / (float)width + eps);
#pragma unroll
    for (int i = 0; i < MAXV; ++i) {
      const int c = (threadIdx.x + 256 * i) * 4;
      if (c < width) {
#pragma unroll
        for (int j = 0; j < 4; ++j) dst[c + j] = from_float<TO>(v[i][j] * inv * w[i][j]);
      }
    }
    return;
  }
  float sum = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = src[i];
    sum += v * v;
  }
  sum = block_sum(sum, scratch);
  const float inv = 1.0f / sqrtf(sum / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) dst[i] = from_float<TO>(src[i] * inv * weight[i]);
}

extern "C" int vk_rmsnorm(const float* x, const float* weight, const int* rows, void* out, int out_dtype,
                          int num_rows, int width, float eps, void* stream) {
  if (num_rows <= 0) return 0;
  if (width <= 0) return VK_BAD_ARGUMENT;
  hipStream_t s = (hipStream_t)stream;
  if (out_dtype == DT_F32)
    rmsnorm_kernel<float><<<num_rows, 256, 0, s>>>(x, weight, rows, (float*)out, width, eps);
  else if (out_dtype == DT_BF16)
    rmsnorm_kernel<bf16_t><<<num_rows, 256, 0, s>>>(x, weight, rows, (bf16_t*)out, width, eps);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// One wave per (token, head), four heads to a workgroup: grid (tokens, ceil((heads + 2 * kv_heads) / 4));
// the last kv_heads of a row are the value heads. `qkv` row layout: [heads*hd | kv_heads*hd | kv_heads*hd].
// The first `rotary_dim` dims of every q and k head are rotated in place (angles in 32-bit:
// float(pos) * inv_freq[i]); then the token's K and V rows go to the paged cache. K pages are
// [page, kv_head, slot, hd]; V pages are transposed, [page, kv_head, hd, slot], so that the
// attention kernels read consecutive positions of one output dim. A token whose page id is
// negative writes nothing to the cache.
// Sines and cosines of a step's rotation angles, once for all heads and all layers that share the
// frequencies: out[t * half + i] = (sin, cos)(float(pos_t) * inv_freq[i]), the same expression in the same
// precision as rope_kvwrite_kernel evaluates without a table (the reference keeps one table per position for
// all layers, crates/vipera-backend-cpu/src/model.rs:4174-4181).
__global__ void rope_angles_kernel(const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                   float2* __restrict__ out, int num_tokens, int half) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)num_tokens * half) return;
  const int t = (int)(idx / half), i = (int)(idx % half);
  float sn, cs;
  sincosf((float)positions[t] * inv_freq[i], &sn, &cs);
  out[idx] = make_float2(sn, cs);
}

extern "C" int vk_rope_angles(const int* positions, const float* inv_freq, int half, int num_tokens, float* out,
                              void* stream) {
  if (num_tokens <= 0 || half <= 0) return 0;
  const long long total = (long long)num_tokens * half;
  if (total > 0x7fffffffLL * 256) return VK_UNSUPPORTED_SIZE;
  rope_angles_kernel<<<(unsigned)((total + 255) / 256), 256, 0, (hipStream_t)stream>>>(positions, inv_freq,
                                                                                        (float2*)out, num_tokens, half);
  VK_LAUNCH_CHECK();
  return 0;
}

constexpr int ROPE_HEADS_PER_BLOCK = 4;  // one wave per head
template <typename T>
__global__ __launch_bounds__(ROPE_HEADS_PER_BLOCK * 64) void rope_kvwrite_kernel(
    T* __restrict__ qkv, const int* __restrict__ positions,
                                                          const float* __restrict__ inv_freq,
                                                          const float2* __restrict__ angles, int rotary_dim,
                                                          T* __restrict__ k_cache, T* __restrict__ v_cache,
                                                          const int* __restrict__ entry_of_token,
                                                          const int* __restrict__ block_table, int table_width,
                                                          int block_size, int heads, int kv_heads, int hd,
                                                          int total_heads) {
  const int t = blockIdx.x, head = blockIdx.y * ROPE_HEADS_PER_BLOCK + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (head >= total_heads) return;
  const int pos = positions[t];
  T* h = qkv + (size_t)t * (heads + 2 * kv_heads) * hd + (size_t)head * hd;
  const bool is_q = head < heads, is_k = !is_q && head < heads + kv_heads;
  const int half = rotary_dim / 2;
  int page = -1;
  if (!is_q && k_cache != nullptr) page = block_table[(size_t)entry_of_token[t] * table_width + pos / block_size];
  const int slot = pos % block_size;
  if (is_q || is_k) {
    const int kvh = head - heads;
    const size_t k_at = is_k && page >= 0 ? (((size_t)page * kv_heads + kvh) * block_size + slot) * hd : 0;
    for (int i = lane; i < hd; i += 64) {
      if (i < half) {
        float sn, cs;
        if (angles) {
          const float2 sc = angles[(size_t)t * half + i];
          sn = sc.x;
          cs = sc.y;
        } else {
          sincosf((float)pos * inv_freq[i], &sn, &cs);
        }
        const float lo = to_float<T>(h[i]), hi = to_float<T>(h[i + half]);
        const T a = from_float<T>(lo * cs - hi * sn), b = from_float<T>(lo * sn + hi * cs);
        h[i] = a;
        h[i + half] = b;
        if (is_k && page >= 0) {
          k_cache[k_at + i] = a;
          k_cache[k_at + i + half] = b;
        }
      } else if (i >= rotary_dim && is_k && page >= 0) {
        k_cache[k_at + i] = h[i];
      }
    }
  } else if (page >= 0) {
    const int kvh = head - heads - kv_heads;
    const size_t v_at = (((size_t)page * kv_heads + kvh) * hd) * block_size + slot;
    for (int i = lane; i < hd; i += 64) v_cache[v_at + (size_t)i * block_size] = h[i];
  }
}

// The same work with 16 bytes per access, for steps of many tokens (the sines come from the step's table): a
// workgroup owns ROPE_GROUP consecutive tokens of the batch, a wave one of them. A lane owns V consecutive dims
// (V = 8 bfloat16 or 4 floats) in the first half of the rotated dims of a q or k head and their partners half a
// rotation width further on; with 64 lanes a wave covers 64 / (half / V) heads at a time, one contiguous stretch of
// the token's row, and keeps its sines across the heads where its chunk stays the same. Dims of a key head past
// the rotated ones are copied to the cache. Value heads: where the group's tokens are eight consecutive positions
// of one request that begin at a multiple of eight (the inside of a prompt's portion), a thread takes V dims of
// all eight tokens, transposes them in registers and writes, per dim, the eight slots of the transposed page as
// one stretch (the 7B prompt of 2,048 tokens: 131,072 stores of 16 bytes instead of a million of two); any other
// group scatters element by element. Per element the arithmetic is that of rope_kvwrite_kernel. Needs head
// width, rotated width and its half to be multiples of V.
constexpr int ROPE_GROUP = 8;
template <typename T>
__global__ __launch_bounds__(ROPE_GROUP * 64) void rope_kvwrite_vector_kernel(
    T* __restrict__ qkv, const int* __restrict__ positions, const float2* __restrict__ angles, int rotary_dim,
    T* __restrict__ k_cache, T* __restrict__ v_cache, const int* __restrict__ entry_of_token,
    const int* __restrict__ block_table, int table_width, int block_size, int heads, int kv_heads, int hd,
    int num_tokens) {
  constexpr int V = 16 / (int)sizeof(T);
  typedef T vec_t __attribute__((ext_vector_type(V)));
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t0 = blockIdx.x * ROPE_GROUP, t = t0 + wave;
  const int half = rotary_dim / 2, row = (heads + 2 * kv_heads) * hd;
  if (t < num_tokens) {
    const int pos = positions[t];
    int page = -1;
    if (k_cache != nullptr) page = block_table[(size_t)entry_of_token[t] * table_width + pos / block_size];
    const int slot = pos % block_size;
    T* token = qkv + (size_t)t * row;
    const int chunks = half / V, items = (heads + kv_heads) * chunks;
    const bool same_chunk = 64 % chunks == 0;  // then u % chunks is the same in every round
    float sn[V], cs[V];
    for (int u = lane; u < items; u += 64) {
      const int head = u / chunks, i0 = (u % chunks) * V;
      if (!same_chunk || u == lane) {
#pragma unroll
        for (int j = 0; j < V; ++j) {
          const float2 sc = angles[(size_t)t * half + i0 + j];
          sn[j] = sc.x;
          cs[j] = sc.y;
        }
      }
      T* h = token + (size_t)head * hd;
      const vec_t lo = *(const vec_t*)(h + i0), hi = *(const vec_t*)(h + i0 + half);
      vec_t a, b;
#pragma unroll
      for (int j = 0; j < V; ++j) {
        const float l = to_float<T>(lo[j]), w = to_float<T>(hi[j]);
        a[j] = from_float<T>(l * cs[j] - w * sn[j]);
        b[j] = from_float<T>(l * sn[j] + w * cs[j]);
      }
      *(vec_t*)(h + i0) = a;
      *(vec_t*)(h + i0 + half) = b;
      if (head >= heads && page >= 0) {
        T* at = k_cache + (((size_t)page * kv_heads + (head - heads)) * block_size + slot) * hd;
        *(vec_t*)(at + i0) = a;
        *(vec_t*)(at + i0 + half) = b;
      }
    }
    if (rotary_dim < hd && page >= 0) {  // the dims of the key heads that are not rotated
      const int tail = (hd - rotary_dim) / V;
      for (int u = lane; u < kv_heads * tail; u += 64) {
        const int kvh = u / tail, i0 = rotary_dim + (u % tail) * V;
        *(vec_t*)(k_cache + (((size_t)page * kv_heads + kvh) * block_size + slot) * hd + i0) =
            *(const vec_t*)(token + (size_t)(heads + kvh) * hd + i0);
      }
    }
  }
  if (k_cache == nullptr) return;
  // the value heads of the group's tokens
  const int v_chunks = hd / V, v_items = kv_heads * v_chunks;
  bool whole = t0 + ROPE_GROUP <= num_tokens && (block_size & 7) == 0;
  int first = 0, entry = 0;
  if (whole) {
    first = positions[t0];
    entry = entry_of_token[t0];
    whole = (first & 7) == 0;
#pragma unroll
    for (int j = 1; j < ROPE_GROUP; ++j)
      whole = whole && positions[t0 + j] == first + j && entry_of_token[t0 + j] == entry;
  }
  if (whole) {
    const int page = block_table[(size_t)entry * table_width + first / block_size];
    if (page < 0) return;
    const int slot = first % block_size;
    for (int u = threadIdx.x; u < v_items; u += ROPE_GROUP * 64) {
      const int kvh = u / v_chunks, i0 = (u % v_chunks) * V;
      vec_t of_token[ROPE_GROUP];
#pragma unroll
      for (int j = 0; j < ROPE_GROUP; ++j)
        of_token[j] = *(const vec_t*)(qkv + (size_t)(t0 + j) * row + (size_t)(heads + kv_heads + kvh) * hd + i0);
      T* at = v_cache + (((size_t)page * kv_heads + kvh) * hd + i0) * block_size + slot;
#pragma unroll
      for (int d = 0; d < V; ++d)
#pragma unroll
        for (int part = 0; part < ROPE_GROUP / V; ++part) {
          vec_t slots;
#pragma unroll
          for (int j = 0; j < V; ++j) slots[j] = of_token[part * V + j][d];
          *(vec_t*)(at + (size_t)d * block_size + part * V) = slots;
        }
    }
    return;
  }
  const int count = min(ROPE_GROUP, num_tokens - t0);
  for (int u = threadIdx.x; u < count * v_items; u += ROPE_GROUP * 64) {
    const int tt = t0 + u / v_items, item = u % v_items;
    const int kvh = item / v_chunks, i0 = (item % v_chunks) * V;
    const int pos = positions[tt];
    const int page = block_table[(size_t)entry_of_token[tt] * table_width + pos / block_size];
    if (page < 0) continue;
    const vec_t v = *(const vec_t*)(qkv + (size_t)tt * row + (size_t)(heads + kv_heads + kvh) * hd + i0);
    T* at = v_cache + (((size_t)page * kv_heads + kvh) * hd + i0) * block_size + pos % block_size;
#pragma unroll
    for (int j = 0; j < V; ++j) at[(size_t)j * block_size] = v[j];
  }
}

// `angles` (may be null): the step's table from vk_rope_angles, [num_tokens, rotary_dim / 2] pairs.
extern "C" int vk_rope_kvwrite(void* qkv, int dtype, const int* positions, const float* inv_freq, const float* angles,
                               int rotary_dim, void* k_cache, void* v_cache, const int* entry_of_token, const int* block_table,
                               int table_width, int block_size, int num_tokens, int heads, int kv_heads, int hd,
                               void* stream) {
  if (num_tokens <= 0) return 0;
  if (hd <= 0 || heads <= 0 || kv_heads <= 0 || rotary_dim < 0 || rotary_dim > hd || (rotary_dim & 1))
    return VK_BAD_ARGUMENT;
  if (k_cache && (block_size <= 0 || table_width <= 0)) return VK_BAD_ARGUMENT;
  if (heads + 2 * kv_heads > 65535) return VK_UNSUPPORTED_SIZE;
  hipStream_t s = (hipStream_t)stream;
  const int total_heads = heads + (k_cache ? 2 : 1) * kv_heads;  // without a cache the value heads have nothing to do
  {  // 16 bytes per thread where the widths allow it and the sines come from the step's table (a step of many
     // tokens); computing eight sines in a row per thread is slower than one per lane (measured with 8 tokens)
    const int v = dtype == DT_F32 ? 4 : 8;
    const bool aligned = (((uintptr_t)qkv | (uintptr_t)k_cache | (uintptr_t)v_cache) & 15) == 0;
    if ((dtype == DT_F32 || dtype == DT_BF16) && angles != nullptr && aligned && rotary_dim > 0 && hd % v == 0 && rotary_dim % v == 0 &&
        (rotary_dim / 2) % v == 0) {
      const unsigned groups = (unsigned)((num_tokens + ROPE_GROUP - 1) / ROPE_GROUP);
      if (dtype == DT_F32)
        rope_kvwrite_vector_kernel<float><<<groups, ROPE_GROUP * 64, 0, s>>>(
            (float*)qkv, positions, (const float2*)angles, rotary_dim, (float*)k_cache, (float*)v_cache, entry_of_token,
            block_table, table_width, block_size, heads, kv_heads, hd, num_tokens);
      else
        rope_kvwrite_vector_kernel<bf16_t><<<groups, ROPE_GROUP * 64, 0, s>>>(
            (bf16_t*)qkv, positions, (const float2*)angles, rotary_dim, (bf16_t*)k_cache, (bf16_t*)v_cache,
            entry_of_token, block_table, table_width, block_size, heads, kv_heads, hd, num_tokens);
      VK_LAUNCH_CHECK();
      return 0;
    }
  }
  const dim3 grid(num_tokens, (total_heads + ROPE_HEADS_PER_BLOCK - 1) / ROPE_HEADS_PER_BLOCK);
  constexpr int threads = ROPE_HEADS_PER_BLOCK * 64;
  if (dtype == DT_F32)
    rope_kvwrite_kernel<float><<<grid, threads, 0, s>>>((float*)qkv, positions, inv_freq, (const float2*)angles,
                                                        rotary_dim, (float*)k_cache,
                                                        (float*)v_cache, entry_of_token, block_table, table_width,
                                                        block_size, heads, kv_heads, hd, total_heads);
  else if (dtype == DT_BF16)
    rope_kvwrite_kernel<bf16_t><<<grid, threads, 0, s>>>((bf16_t*)qkv, positions, inv_freq, (const float2*)angles,
                                                         rotary_dim,
                                                         (bf16_t*)k_cache, (bf16_t*)v_cache, entry_of_token,
                                                         block_table, table_width, block_size, heads, kv_heads, hd,
                                                         total_heads);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// out[t, i] = up * silu(gate); math in 32-bit. Two layouts of a gate_up row: [gate | up] halves, or
// `interleaved` in groups of 16 (gate of outputs 16 p .. 16 p + 15 at columns 32 p .., their up values
// at columns 32 p + 16 ..), which is what the fused matrix-core product of the feed-forward wants.
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gate_up, T* __restrict__ out, int inter, long long total,
                              int interleaved) {
  for (long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x; idx < total;
       idx += (long long)gridDim.x * blockDim.x) {
    const long long t = idx / inter;
    const int i = (int)(idx - t * inter);
    const T* row = gate_up + t * 2 * inter;
    const int gi = interleaved ? (i / 16) * 32 + (i % 16) : i;
    const int ui = interleaved ? gi + 16 : inter + i;
    const float g = to_float<T>(row[gi]), u = to_float<T>(row[ui]);
    out[idx] = from_float<T>(u * (g / (1.0f + expf(-g))));
  }
}

extern "C" int vk_swiglu(const void* gate_up, void* out, int dtype, int num_tokens, int inter, int interleaved,
                         void* stream) {
  if (num_tokens <= 0) return 0;
  if (inter <= 0 || (interleaved && (inter & 15))) return VK_BAD_ARGUMENT;
  const long long total = (long long)num_tokens * inter;
  long long blocks = (total + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32)
    swiglu_kernel<float><<<(int)blocks, 256, 0, s>>>((const float*)gate_up, (float*)out, inter, total, interleaved);
  else if (dtype == DT_BF16)
    swiglu_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((const bf16_t*)gate_up, (bf16_t*)out, inter, total, interleaved);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------------------------
// Counter-based normal fill: element i of a stream is a function of (key, i) alone.
//   z = mix(key + (i+1)*GOLDEN); u1 = (hi32(z)+0.5)/2^32; u2 = lo32(z)/2^32;
//   n = sqrt(-2 ln u1) * cos(2 pi u2) in 64-bit; out = offset + std * n
template <typename T>
__global__ void fill_normal_kernel(T* __restrict__ out, long long count, unsigned long long key, float std_,
                                   float offset) {
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < count;
       i += (long long)gridDim.x * blockDim.x) {
    unsigned long long z = key + (unsigned long long)(i + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z = z ^ (z >> 31);
    const double u1 = ((double)(z >> 32) + 0.5) / 4294967296.0;
    const double u2 = (double)(z & 0xFFFFFFFFull) / 4294967296.0;
    const double n = sqrt(-2.0 * log(u1)) * cos(6.283185307179586476925286766559 * u2);
    const double scaled = n * (double)std_;
    out[i] = from_float<T>((float)(offset != 0.f ? (double)offset + scaled : scaled));
  }
}

extern "C" int vk_fill_normal(void* out, int dtype, long long count, unsigned long long key, float std_,
                              float offset, void* stream) {
  if (count <= 0) return 0;
  long long blocks = (count + 255) / 256;
  if (blocks > 16384) blocks = 16384;
  hipStream_t s = (hipStream_t)stream;
  if (dtype == DT_F32)
    fill_normal_kernel<float><<<(int)blocks, 256, 0, s>>>((float*)out, count, key, std_, offset);
  else if (dtype == DT_BF16)
    fill_normal_kernel<bf16_t><<<(int)blocks, 256, 0, s>>>((bf16_t*)out, count, key, std_, offset);
  else
    return VK_BAD_ARGUMENT;
  VK_LAUNCH_CHECK();
  return 0;
}
