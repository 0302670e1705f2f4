// Plain C++ twins of the engine's kernels: the same parameter lists as the `vk_*` entry points (the stream is
// ignored, pointers are host memory), straight loops, one formula at a time, double sums where the kernels sum in
// 32-bit. Nothing here is on the product path; the tests call these through ctypes and compare each kernel with its
// twin, and run a whole tiny model through them to compare with the Python plain implementation.
//
// Formulas as the reference computes them (crates/vipera-backend-cpu/src/model.rs unless another file is named):
//   embedding 607-616, RMSNorm 4282-4288, products with the bias after the product 1005-1031, rotation 4192-4251,
//   cache write 1495-1542, attention 1811-1857 (window 2509), SwiGLU 4368-4374, residual sums 666-668 and 672-680;
//   sampling crates/vipera-sampler/src/lib.rs 135-248 and 596-616.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

namespace {
constexpr int DT_F32 = 0, DT_BF16 = 1;
constexpr int BAD_ARGUMENT = -1;

float bf16_to_float(uint16_t v) {
  const uint32_t bits = (uint32_t)v << 16;
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

// round to nearest, ties to even; NaN stays NaN
uint16_t float_to_bf16(float f) {
  uint32_t bits;
  std::memcpy(&bits, &f, 4);
  if ((bits & 0x7f800000u) == 0x7f800000u && (bits & 0x007fffffu)) return (uint16_t)((bits >> 16) | 0x0040u);
  bits += 0x7fffu + ((bits >> 16) & 1u);
  return (uint16_t)(bits >> 16);
}

float load(const void* p, int dtype, size_t i) {
  return dtype == DT_F32 ? ((const float*)p)[i] : bf16_to_float(((const uint16_t*)p)[i]);
}

void store(void* p, int dtype, size_t i, float v) {
  if (dtype == DT_F32) ((float*)p)[i] = v;
  else ((uint16_t*)p)[i] = float_to_bf16(v);
}

bool known(int dtype) { return dtype == DT_F32 || dtype == DT_BF16; }

// C[m, n] (+)= sum_k A[m, k] * W[n, k] + bias[n]; the sum in double, rounded once to 32-bit
void product(const void* A, int a_dtype, const void* W, int w_dtype, const float* bias, void* C, int c_dtype, int M,
             int N, int K, long long lda, long long ldc, bool accumulate) {
  for (int m = 0; m < M; ++m)
    for (int n = 0; n < N; ++n) {
      double sum = 0.0;
      for (int k = 0; k < K; ++k)
        sum += (double)load(A, a_dtype, (size_t)m * lda + k) * (double)load(W, w_dtype, (size_t)n * K + k);
      float v = (float)sum;
      if (bias) v += bias[n];
      if (accumulate) v += load(C, c_dtype, (size_t)m * ldc + n);
      store(C, c_dtype, (size_t)m * ldc + n, v);
    }
}

// One token's attention for one query head: positions [lo, pos] of its request's pages. Plain softmax: scores,
// their maximum, weights, normalised before the multiply-add as the reference does (model.rs:1840-1857).
void attend(const void* q_row, const void* k_cache, const void* v_cache, int dtype, const int* table, int block_size,
            int kv_heads, int kvh, int hd, float scale, int pos, int window, void* out_row) {
  const int hi = pos + 1, lo = (window > 0 && hi > window) ? hi - window : 0;
  std::vector<double> score(hi - lo);
  double peak = -std::numeric_limits<double>::infinity();
  for (int p = lo; p < hi; ++p) {
    const size_t k_at = (((size_t)table[p / block_size] * kv_heads + kvh) * block_size + p % block_size) * hd;
    double dot = 0.0;
    for (int d = 0; d < hd; ++d) dot += (double)load(q_row, dtype, d) * (double)load(k_cache, dtype, k_at + d);
    score[p - lo] = dot * (double)scale;
    peak = std::max(peak, score[p - lo]);
  }
  double total = 0.0;
  for (double& s : score) {
    s = std::exp(s - peak);
    total += s;
  }
  for (int d = 0; d < hd; ++d) {
    double sum = 0.0;
    for (int p = lo; p < hi; ++p) {
      const size_t v_at = (((size_t)table[p / block_size] * kv_heads + kvh) * hd + d) * block_size + p % block_size;
      sum += (score[p - lo] / total) * (double)load(v_cache, dtype, v_at);
    }
    store(out_row, dtype, d, (float)sum);
  }
}

bool finite(float v) { return std::isfinite(v); }
}  // namespace

// --- row-wise and element-wise -------------------------------------------------------------------------------
extern "C" int plain_embed_gather(const void* table, int table_dtype, const int* tokens, const int* source,
                                  const int* sampled, float* out, int num_tokens, int width, int vocab, void*) {
  if (num_tokens <= 0) return 0;
  if (width <= 0 || vocab <= 0 || !known(table_dtype) || (source && !sampled)) return BAD_ARGUMENT;
  for (int t = 0; t < num_tokens; ++t) {
    int token = tokens[t];
    if (source && source[t] >= 0) token = sampled[source[t]];
    if (token < 0 || token >= vocab) token = 0;
    for (int i = 0; i < width; ++i) out[(size_t)t * width + i] = load(table, table_dtype, (size_t)token * width + i);
  }
  return 0;
}

extern "C" int plain_rmsnorm(const float* x, const float* weight, const int* rows, void* out, int out_dtype,
                             int num_rows, int width, float eps, void*) {
  if (num_rows <= 0) return 0;
  if (width <= 0 || !known(out_dtype)) return BAD_ARGUMENT;
  for (int r = 0; r < num_rows; ++r) {
    const float* src = x + (size_t)(rows ? rows[r] : r) * width;
    double sum = 0.0;
    for (int i = 0; i < width; ++i) sum += (double)src[i] * (double)src[i];
    const float inv = 1.0f / std::sqrt((float)(sum / width) + eps);
    for (int i = 0; i < width; ++i) store(out, out_dtype, (size_t)r * width + i, (src[i] * inv) * weight[i]);
  }
  return 0;
}

extern "C" int plain_rope_angles(const int* positions, const float* inv_freq, int half, int num_tokens, float* out,
                                 void*) {
  for (int t = 0; t < num_tokens; ++t)
    for (int i = 0; i < half; ++i) {
      const float angle = (float)positions[t] * inv_freq[i];   // 32-bit, as the reference rounds it
      out[((size_t)t * half + i) * 2] = (float)std::sin((double)angle);
      out[((size_t)t * half + i) * 2 + 1] = (float)std::cos((double)angle);
    }
  return 0;
}

extern "C" int plain_rope_kvwrite(void* qkv, int dtype, const int* positions, const float* inv_freq,
                                  const float* angles, int rotary_dim, void* k_cache, void* v_cache,
                                  const int* entry_of_token, const int* block_table, int table_width, int block_size,
                                  int num_tokens, int heads, int kv_heads, int hd, void*) {
  if (num_tokens <= 0) return 0;
  if (!known(dtype) || hd <= 0 || heads <= 0 || kv_heads <= 0 || rotary_dim < 0 || rotary_dim > hd || (rotary_dim & 1))
    return BAD_ARGUMENT;
  if (k_cache && (block_size <= 0 || table_width <= 0)) return BAD_ARGUMENT;
  const int half = rotary_dim / 2, row = (heads + 2 * kv_heads) * hd;
  for (int t = 0; t < num_tokens; ++t) {
    const int pos = positions[t];
    for (int head = 0; head < heads + kv_heads; ++head)   // q heads, then k heads
      for (int i = 0; i < half; ++i) {
        float sn, cs;
        if (angles) {
          sn = angles[((size_t)t * half + i) * 2];
          cs = angles[((size_t)t * half + i) * 2 + 1];
        } else {
          const float angle = (float)pos * inv_freq[i];
          sn = (float)std::sin((double)angle);
          cs = (float)std::cos((double)angle);
        }
        const size_t at = (size_t)t * row + (size_t)head * hd + i;
        const float lo = load(qkv, dtype, at), hi = load(qkv, dtype, at + half);
        store(qkv, dtype, at, lo * cs - hi * sn);
        store(qkv, dtype, at + half, lo * sn + hi * cs);
      }
    if (!k_cache) continue;
    const int page = block_table[(size_t)entry_of_token[t] * table_width + pos / block_size];
    if (page < 0) continue;
    const int slot = pos % block_size;
    for (int kvh = 0; kvh < kv_heads; ++kvh)
      for (int d = 0; d < hd; ++d) {
        const float k = load(qkv, dtype, (size_t)t * row + (size_t)(heads + kvh) * hd + d);
        const float v = load(qkv, dtype, (size_t)t * row + (size_t)(heads + kv_heads + kvh) * hd + d);
        store(k_cache, dtype, (((size_t)page * kv_heads + kvh) * block_size + slot) * hd + d, k);
        store(v_cache, dtype, (((size_t)page * kv_heads + kvh) * hd + d) * block_size + slot, v);
      }
  }
  return 0;
}

extern "C" int plain_swiglu(const void* gate_up, void* out, int dtype, int num_tokens, int inter, int interleaved,
                            void*) {
  if (num_tokens <= 0) return 0;
  if (!known(dtype) || inter <= 0 || (interleaved && (inter & 15))) return BAD_ARGUMENT;
  for (int t = 0; t < num_tokens; ++t)
    for (int i = 0; i < inter; ++i) {
      const int gi = interleaved ? (i / 16) * 32 + i % 16 : i;
      const int ui = interleaved ? gi + 16 : inter + i;
      const double g = load(gate_up, dtype, (size_t)t * 2 * inter + gi), u = load(gate_up, dtype, (size_t)t * 2 * inter + ui);
      store(out, dtype, (size_t)t * inter + i, (float)(u * (g / (1.0 + std::exp(-g)))));
    }
  return 0;
}

// --- products --------------------------------------------------------------------------------------------------
extern "C" int plain_gemm_generic(const void* A, int a_dtype, const void* W, int w_dtype, const float* bias, void* C,
                                  int c_dtype, int M, int N, int K, long long lda, long long ldc, int accumulate,
                                  void*) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || !known(a_dtype) || !known(w_dtype) || !known(c_dtype) || lda < K || ldc < N) return BAD_ARGUMENT;
  product(A, a_dtype, W, w_dtype, bias, C, c_dtype, M, N, K, lda, ldc, accumulate != 0);
  return 0;
}

// the 32-bit weight stream for up to 64 tokens; the workspace shapes the kernel's work only
extern "C" int plain_gemm_stream(const float* A, const float* W, const float* bias, void* C, int c_dtype, int M, int N,
                                 int K, long long lda, long long ldc, int accumulate, float*, long long, void*) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || M > 64 || !known(c_dtype) || lda < K || ldc < N || (accumulate && c_dtype != DT_F32)) return BAD_ARGUMENT;
  product(A, DT_F32, W, DT_F32, bias, C, c_dtype, M, N, K, lda, ldc, accumulate != 0);
  return 0;
}

extern "C" int plain_gemm_bf16(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N,
                               int K, long long lda, long long ldc, int accumulate, int, int, float*, long long,
                               void*) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || !known(c_dtype) || lda < K || ldc < N || (accumulate && c_dtype != DT_F32)) return BAD_ARGUMENT;
  product(A, DT_BF16, W, DT_BF16, bias, C, c_dtype, M, N, K, lda, ldc, accumulate != 0);
  return 0;
}

extern "C" int plain_gemm_bf16_mid(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N,
                                   int K, long long lda, long long ldc, int accumulate, int, int, float*, long long,
                                   void*) {
  return plain_gemm_bf16(A, W, bias, C, c_dtype, M, N, K, lda, ldc, accumulate, 0, 0, nullptr, 0, nullptr);
}

// out[m, 16 p + j] = up * silu(gate), gate = row 32 p + j and up = row 32 p + 16 + j of the fused weight
extern "C" int plain_gemm_bf16_gated(const void* A, const void* W, void* C, int M, int N, int K, long long lda,
                                     long long ldc, int, void*) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || (N & 31) || ldc < N / 2) return BAD_ARGUMENT;
  for (int m = 0; m < M; ++m)
    for (int i = 0; i < N / 2; ++i) {
      const int gate_row = (i / 16) * 32 + i % 16, up_row = gate_row + 16;
      double gate = 0.0, up = 0.0;
      for (int k = 0; k < K; ++k) {
        const double a = load(A, DT_BF16, (size_t)m * lda + k);
        gate += a * (double)load(W, DT_BF16, (size_t)gate_row * K + k);
        up += a * (double)load(W, DT_BF16, (size_t)up_row * K + k);
      }
      store(C, DT_BF16, (size_t)m * ldc + i, (float)(up * (gate / (1.0 + std::exp(-gate)))));
    }
  return 0;
}

// The fused q/k/v product: the product in bfloat16, then the rotation and the cache write on its output. With
// `sumsq`, A is x * gain of a norm whose division is still due: the product's sums are divided by the root mean
// square that the `norm_groups` sums of squares give, before the bias.
extern "C" int plain_rope_kvwrite(void* qkv, int dtype, const int* positions, const float* inv_freq,
                                  const float* angles, int rotary_dim, void* k_cache, void* v_cache,
                                  const int* entry_of_token, const int* block_table, int table_width, int block_size,
                                  int num_tokens, int heads, int kv_heads, int hd, void*);
static int qkv_rope(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, long long lda,
                    long long ldc, const int* positions, const float* inv_freq, void* k_cache, void* v_cache,
                    const int* entry_of_token, const int* block_table, int table_width, int block_size, int heads,
                    int kv_heads, int hd, const float* sumsq, int norm_groups, int sumsq_stride, float eps);
extern "C" int plain_gemm_bf16_qkv_rope(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                                        long long lda, long long ldc, const int* positions, const float* inv_freq,
                                        void* k_cache, void* v_cache, const int* entry_of_token, const int* block_table,
                                        int table_width, int block_size, int heads, int kv_heads, int hd,
                                        const float* sumsq, int norm_groups, float eps, void*) {
  return qkv_rope(A, W, bias, C, M, N, K, lda, ldc, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table,
                  table_width, block_size, heads, kv_heads, hd, sumsq, norm_groups, 16, eps);
}
// The same where the kernel splits K over workgroups and takes up to 64 tokens (no difference for the twin).
extern "C" int plain_gemm_bf16_mid_qkv_rope(const void* A, const void* W, const float* bias, void* C, int M, int N, int K,
                                            long long lda, long long ldc, int, int, float*, long long,
                                            const int* positions, const float* inv_freq, void* k_cache, void* v_cache,
                                            const int* entry_of_token, const int* block_table, int table_width,
                                            int block_size, int heads, int kv_heads, int hd, const float* sumsq,
                                            int norm_groups, int sumsq_stride, float eps, void*) {
  return qkv_rope(A, W, bias, C, M, N, K, lda, ldc, positions, inv_freq, k_cache, v_cache, entry_of_token, block_table,
                  table_width, block_size, heads, kv_heads, hd, sumsq, norm_groups, sumsq_stride, eps);
}
static int qkv_rope(const void* A, const void* W, const float* bias, void* C, int M, int N, int K, long long lda,
                    long long ldc, const int* positions, const float* inv_freq, void* k_cache, void* v_cache,
                    const int* entry_of_token, const int* block_table, int table_width, int block_size, int heads,
                    int kv_heads, int hd, const float* sumsq, int norm_groups, int sumsq_stride, float eps) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldc != N || (long long)(heads + 2 * kv_heads) * hd != N) return BAD_ARGUMENT;
  for (int m = 0; m < M; ++m) {
    double inv = 1.0;
    if (sumsq) {
      double squares = 0.0;
      for (int g = 0; g < norm_groups; ++g) squares += (double)sumsq[(size_t)g * sumsq_stride + m];
      inv = 1.0 / std::sqrt(squares / (double)K + (double)eps);
    }
    for (int n = 0; n < N; ++n) {
      double sum = 0.0;
      for (int k = 0; k < K; ++k)
        sum += (double)load(A, DT_BF16, (size_t)m * lda + k) * (double)load(W, DT_BF16, (size_t)n * K + k);
      store(C, DT_BF16, (size_t)m * ldc + n, (float)(sum * inv) + (bias ? bias[n] : 0.f));
    }
  }
  return plain_rope_kvwrite(C, DT_BF16, positions, inv_freq, nullptr, hd, k_cache, v_cache, entry_of_token, block_table,
                            table_width, block_size, M, heads, kv_heads, hd, nullptr);
}

// The residual product that also prepares the norm after it: C += A W^T + bias; scaled = bfloat16(C * gain); the
// sums of squares of the rows of C as one group.
extern "C" int plain_gemm_bf16_follow(const void* A, const void* W, const float* bias, float* C, int M, int N, int K,
                                      long long lda, long long ldc, const float* gain, void* scaled, long long ld_scaled,
                                      float* sumsq, long long sumsq_floats, int* groups, void*) {
  if (M <= 0 || N <= 0 || M > 16 || K <= 0 || lda < K || ldc < N || ld_scaled < N || sumsq_floats < 16) return BAD_ARGUMENT;
  product(A, DT_BF16, W, DT_BF16, bias, C, DT_F32, M, N, K, lda, ldc, true);
  for (int m = 0; m < 16; ++m) sumsq[m] = 0.f;
  for (int m = 0; m < M; ++m) {
    double sum = 0.0;
    for (int n = 0; n < N; ++n) {
      const float x = C[(size_t)m * ldc + n];
      sum += (double)x * (double)x;
      ((uint16_t*)scaled)[(size_t)m * ld_scaled + n] = float_to_bf16(x * gain[n]);
    }
    sumsq[m] = (float)sum;
  }
  *groups = 1;
  return 0;
}

extern "C" int plain_gemm_bf16_follow(const void* A, const void* W, const float* bias, float* C, int M, int N, int K,
                                      long long lda, long long ldc, const float* gain, void* scaled, long long ld_scaled,
                                      float* sumsq, long long sumsq_floats, int* groups, void*);
// The same where the kernel splits K over workgroups (no difference for the twin).
extern "C" int plain_gemm_bf16_mid_follow(const void* A, const void* W, const float* bias, float* C, int M, int N, int K,
                                          long long lda, long long ldc, int, int, float*, long long, const float* gain,
                                          void* scaled, long long ld_scaled, float* sumsq, long long sumsq_floats,
                                          int sumsq_stride, int* groups, void*) {
  if (M <= 0 || N <= 0 || M > sumsq_stride || K <= 0 || lda < K || ldc < N || ld_scaled < N || sumsq_floats < sumsq_stride)
    return BAD_ARGUMENT;
  product(A, DT_BF16, W, DT_BF16, bias, C, DT_F32, M, N, K, lda, ldc, true);
  for (int m = 0; m < sumsq_stride; ++m) sumsq[m] = 0.f;
  for (int m = 0; m < M; ++m) {
    double sum = 0.0;
    for (int n = 0; n < N; ++n) {
      const float x = C[(size_t)m * ldc + n];
      sum += (double)x * (double)x;
      ((uint16_t*)scaled)[(size_t)m * ld_scaled + n] = float_to_bf16(x * gain[n]);
    }
    sumsq[m] = (float)sum;
  }
  *groups = 1;
  return 0;
}

// The gated product on such a scaled input: gate and up divided by the root mean square first.
extern "C" int plain_gemm_bf16_gated_scaled(const void* A, const void* W, void* C, int M, int N, int K, long long lda,
                                            long long ldc, const float* sumsq, int groups, float eps, void*) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || (N & 31) || ldc < N / 2 || groups <= 0) return BAD_ARGUMENT;
  for (int m = 0; m < M; ++m) {
    double squares = 0.0;
    for (int g = 0; g < groups; ++g) squares += (double)sumsq[(size_t)g * 16 + m];
    const double inv = 1.0 / std::sqrt(squares / (double)K + (double)eps);
    for (int i = 0; i < N / 2; ++i) {
      const int gate_row = (i / 16) * 32 + i % 16, up_row = gate_row + 16;
      double gate = 0.0, up = 0.0;
      for (int k = 0; k < K; ++k) {
        const double a = load(A, DT_BF16, (size_t)m * lda + k);
        gate += a * (double)load(W, DT_BF16, (size_t)gate_row * K + k);
        up += a * (double)load(W, DT_BF16, (size_t)up_row * K + k);
      }
      gate *= inv;
      up *= inv;
      store(C, DT_BF16, (size_t)m * ldc + i, (float)(up * (gate / (1.0 + std::exp(-gate)))));
    }
  }
  return 0;
}

// The gated product on the tiled kernel on such a scaled input, for any number of tokens.
extern "C" int plain_gemm_bf16_gated_tile_scaled(const void* A, const void* W, void* C, int M, int N, int K,
                                                 long long lda, long long ldc, const float* sumsq, int groups, int stride,
                                                 float eps, void*) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || (N & 31) || ldc < N / 2 || groups <= 0 || stride < M) return BAD_ARGUMENT;
  for (int m = 0; m < M; ++m) {
    double squares = 0.0;
    for (int g = 0; g < groups; ++g) squares += (double)sumsq[(size_t)g * stride + m];
    const double inv = 1.0 / std::sqrt(squares / (double)K + (double)eps);
    for (int i = 0; i < N / 2; ++i) {
      const int gate_row = (i / 16) * 32 + i % 16, up_row = gate_row + 16;
      double gate = 0.0, up = 0.0;
      for (int k = 0; k < K; ++k) {
        const double a = load(A, DT_BF16, (size_t)m * lda + k);
        gate += a * (double)load(W, DT_BF16, (size_t)gate_row * K + k);
        up += a * (double)load(W, DT_BF16, (size_t)up_row * K + k);
      }
      gate *= inv;
      up *= inv;
      store(C, DT_BF16, (size_t)m * ldc + i, (float)(up * (gate / (1.0 + std::exp(-gate)))));
    }
  }
  return 0;
}

// --- attention over the paged cache ----------------------------------------------------------------------------
extern "C" int plain_attn_generic(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                                  void* out, int dtype, const int* positions, const int* entry_of_token,
                                  const int* block_table, int table_width, int block_size, int num_tokens, int heads,
                                  int kv_heads, int hd, float scale, int window, const int* skip_single_of, void*) {
  if (num_tokens <= 0) return 0;
  if (!known(dtype) || hd <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || block_size <= 0 || window < 0)
    return BAD_ARGUMENT;
  const size_t elem = dtype == DT_F32 ? 4 : 2;
  for (int t = 0; t < num_tokens; ++t) {
    // skip_single_of: the step's entry_start; the token of an entry that holds one token is left alone
    if (skip_single_of && skip_single_of[entry_of_token[t] + 1] - skip_single_of[entry_of_token[t]] == 1) continue;
    for (int h = 0; h < heads; ++h)
      attend((const char*)q + ((size_t)t * q_stride + (size_t)h * hd) * elem, k_cache, v_cache, dtype,
             block_table + (size_t)entry_of_token[t] * table_width, block_size, kv_heads, h / (heads / kv_heads), hd,
             scale, positions[t], window, (char*)out + ((size_t)t * heads * hd + (size_t)h * hd) * elem);
  }
  return 0;
}

// the 32-bit attention of single-token entries; `partial` and `chunks` shape the kernel's work only
extern "C" int plain_attn_decode_f32(const float* q, long long q_stride, const float* k_cache, const float* v_cache,
                                     float* out, float*, const int* entries, int num_entries, const int* entry_start,
                                     const int* entry_first_pos, const int* block_table, int table_width,
                                     int block_size, int heads, int kv_heads, int hd, float scale, int window, int,
                                     void*) {
  if (hd <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || block_size <= 0 || window < 0) return BAD_ARGUMENT;
  for (int e = 0; e < num_entries; ++e) {
    const int entry = entries[e], t = entry_start[entry];
    for (int h = 0; h < heads; ++h)
      attend(q + (size_t)t * q_stride + (size_t)h * hd, k_cache, v_cache, DT_F32,
             block_table + (size_t)entry * table_width, block_size, kv_heads, h / (heads / kv_heads), hd, scale,
             entry_first_pos[entry], window, out + (size_t)t * heads * hd + (size_t)h * hd);
  }
  return 0;
}

// tiles: pairs (entry, first token of the tile within the entry), `tile_tokens` tokens per tile
extern "C" int plain_attn_prefill_f32(const float* q, long long q_stride, const float* k_cache, const float* v_cache,
                                      float* out, const int* tiles, int num_tiles, int tile_tokens,
                                      const int* entry_start, const int* entry_first_pos, const int* block_table,
                                      int table_width, int block_size, int heads, int kv_heads, int hd, float scale,
                                      int window, void*) {
  if (hd <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || block_size <= 0 || window < 0 || tile_tokens <= 0)
    return BAD_ARGUMENT;
  for (int tile = 0; tile < num_tiles; ++tile) {
    const int entry = tiles[2 * tile], off = tiles[2 * tile + 1];
    const int tok0 = entry_start[entry], count = entry_start[entry + 1] - tok0;
    for (int i = off; i < std::min(off + tile_tokens, count); ++i)
      for (int h = 0; h < heads; ++h)
        attend(q + (size_t)(tok0 + i) * q_stride + (size_t)h * hd, k_cache, v_cache, DT_F32,
               block_table + (size_t)entry * table_width, block_size, kv_heads, h / (heads / kv_heads), hd, scale,
               entry_first_pos[entry] + i, window, out + (size_t)(tok0 + i) * heads * hd + (size_t)h * hd);
  }
  return 0;
}

// tiles: pairs (entry, first token of the tile within the entry), 128 tokens per tile; `split`, the workspace and the
// chunking shape the kernel's work only
extern "C" int plain_attn_bf16_prefill(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                                       void* out, const int* tiles, int num_tiles, const int* entry_start,
                                       const int* entry_first_pos, const int* block_table, int table_width,
                                       int block_size, int heads, int kv_heads, int hd, float scale, int window,
                                       int, float*, long long, int, int, void*) {
  if (hd <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || block_size <= 0 || window < 0) return BAD_ARGUMENT;
  for (int tile = 0; tile < num_tiles; ++tile) {
    const int entry = tiles[2 * tile], off = tiles[2 * tile + 1];
    const int tok0 = entry_start[entry], count = entry_start[entry + 1] - tok0;
    for (int i = off; i < std::min(off + 128, count); ++i)
      for (int h = 0; h < heads; ++h)
        attend((const uint16_t*)q + (size_t)(tok0 + i) * q_stride + (size_t)h * hd, k_cache, v_cache, DT_BF16,
               block_table + (size_t)entry * table_width, block_size, kv_heads, h / (heads / kv_heads), hd, scale,
               entry_first_pos[entry] + i, window, (uint16_t*)out + (size_t)(tok0 + i) * heads * hd + (size_t)h * hd);
  }
  return 0;
}

// entries: the entries that hold exactly one token; `partial`, `chunk`, `chunks` and `join` shape the kernel's work only
extern "C" int plain_attn_bf16_decode(const void* q, long long q_stride, const void* k_cache, const void* v_cache,
                                      void* out, float*, const int* entries, int num_entries, const int* entry_start,
                                      const int* entry_first_pos, const int* block_table, int table_width,
                                      int block_size, int heads, int kv_heads, int hd, float scale, int window, int,
                                      int, int dense, int, void*) {
  if (hd <= 0 || heads <= 0 || kv_heads <= 0 || heads % kv_heads || block_size <= 0 || window < 0) return BAD_ARGUMENT;
  for (int e = 0; e < num_entries; ++e) {
    // dense: entry e is the e-th single-token entry and holds token e
    const int entry = dense ? e : entries[e], t = dense ? e : entry_start[entry];
    for (int h = 0; h < heads; ++h)
      attend((const uint16_t*)q + (size_t)t * q_stride + (size_t)h * hd, k_cache, v_cache, DT_BF16,
             block_table + (size_t)entry * table_width, block_size, kv_heads, h / (heads / kv_heads), hd, scale,
             entry_first_pos[entry], window, (uint16_t*)out + (size_t)t * heads * hd + (size_t)h * hd);
  }
  return 0;
}

// --- sampling --------------------------------------------------------------------------------------------------
// One token per row of logits. temperature 0: argmax over finite logits, ties to the lowest id. Otherwise the
// reference's cuts (candidates by logit descending then id ascending; top_k; top_p against the mass of every finite
// logit; min_p against the best weight) and, as the kernel documents for itself, the draw walks the kept tokens in
// id order: the first whose running mass exceeds u * kept mass. A row without a finite logit gives -1.
// The uniform of a row is uniform[r], or with a slot table the next output of the xorshift64* generator whose state
// sits in the row's slot (crates/vipera-sampler/src/rng.rs:13-57), seeded first where `reseed` says so; a greedy row
// does not draw; the row's position is recorded beside the state.
extern "C" int plain_sample(const float* logits, int num_rows, int vocab, const float* temperature, const int* top_k,
                            const float* top_p, const float* min_p, const double* uniform, int* out, float*, int*, int,
                            const int* slot, const int* position, const int* reseed,
                            const unsigned long long* seed_state, unsigned long long* slot_table, int num_slots, void*) {
  if (num_rows <= 0) return 0;
  if (vocab <= 0) return BAD_ARGUMENT;
  if (!slot_table && !uniform) return BAD_ARGUMENT;
  for (int r = 0; r < num_rows; ++r) {
    const float* row = logits + (size_t)r * vocab;
    double u = uniform ? uniform[r] : 0.0;
    if (slot_table && slot[r] >= 0 && slot[r] < num_slots) {
      unsigned long long state = reseed[r] ? seed_state[r] : slot_table[2 * slot[r]];
      if (temperature[r] > 0.f) {
        state ^= state >> 12;
        state ^= state << 25;
        state ^= state >> 27;
        u = (double)((state * 0x2545F4914F6CDD1Dull) >> 11) / 9007199254740992.0;
      }
      slot_table[2 * slot[r]] = state;
      slot_table[2 * slot[r] + 1] = (unsigned long long)(long long)position[r];
    }
    std::vector<int> order;
    for (int i = 0; i < vocab; ++i)
      if (finite(row[i])) order.push_back(i);
    if (order.empty()) {
      out[r] = -1;
      continue;
    }
    std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return row[a] > row[b]; });
    if (temperature[r] <= 0.f) {
      out[r] = order[0];
      continue;
    }
    const float scale = 1.0f / temperature[r], peak = row[order[0]] * scale;
    double total = 0.0;
    for (int i : order) total += std::exp((double)(row[i] * scale - peak));
    size_t keep = top_k[r] > 0 ? std::min<size_t>(top_k[r], order.size()) : order.size();
    std::vector<double> weight(keep);
    for (size_t j = 0; j < keep; ++j) weight[j] = std::exp((double)(row[order[j]] * scale - peak));
    const double target_mass = (double)top_p[r] * total;
    double running = 0.0;
    for (size_t j = 0; j < keep; ++j) {
      running += weight[j];
      if (running >= target_mass) {
        keep = j + 1;
        break;
      }
    }
    const double threshold = (double)min_p[r] * weight[0];
    std::vector<std::pair<int, double>> kept;
    for (size_t j = 0; j < keep; ++j)
      if (weight[j] >= threshold) kept.push_back({order[j], weight[j]});
    std::sort(kept.begin(), kept.end());   // by id
    double mass = 0.0;
    for (auto& kv : kept) mass += kv.second;
    const double target = u * mass;
    running = 0.0;
    out[r] = kept.back().first;
    for (auto& kv : kept) {
      running += kv.second;
      if (target < running) {
        out[r] = kv.first;
        break;
      }
    }
  }
  return 0;
}

// (row, token, count) triples, unique per (row, token)
extern "C" int plain_penalize(float* logits, int vocab, const int* rows, const int* tokens, const int* counts,
                              const float* repetition, const float* presence, const float* frequency, int n, void*) {
  for (int i = 0; i < n; ++i) {
    const int row = rows[i], token = tokens[i];
    if (token < 0 || token >= vocab) continue;
    float v = logits[(size_t)row * vocab + token];
    if (repetition[row] != 1.0f) v = v > 0.f ? v / repetition[row] : v * repetition[row];
    logits[(size_t)row * vocab + token] = v - (presence[row] + frequency[row] * (float)counts[i]);
  }
  return 0;
}

extern "C" int plain_logit_bias(float* logits, int vocab, const int* rows, const int* tokens, const float* values,
                                int n, void*) {
  for (int i = 0; i < n; ++i)
    if (tokens[i] >= 0 && tokens[i] < vocab) logits[(size_t)rows[i] * vocab + tokens[i]] += values[i];
  return 0;
}

// for the conversion test: all 65,536 patterns both ways
extern "C" void plain_bf16_to_float(const uint16_t* in, float* out, int n) {
  for (int i = 0; i < n; ++i) out[i] = bf16_to_float(in[i]);
}
extern "C" void plain_float_to_bf16(const float* in, uint16_t* out, int n) {
  for (int i = 0; i < n; ++i) out[i] = float_to_bf16(in[i]);
}
