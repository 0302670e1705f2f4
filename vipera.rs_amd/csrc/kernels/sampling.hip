// Sampling on the device: logit penalties, greedy argmax, and temperature sampling with the
// top-k, top-p and min-p cuts. One workgroup of 1024 threads per row of logits.
//
// Meaning of the options as in the reference (crates/vipera-sampler/src/lib.rs):
//   greedy        argmax over finite logits, ties to the lowest id (135-156)
//   temperature   weights exp(l/T - peak), peak = best l/T; the denominator is the mass of every
//                 finite logit (172-203)
//   top_k         keep the k best by (logit descending, id ascending); 0 keeps all (176-186, 440-444)
//   top_p         keep the shortest head whose mass reaches top_p * total mass (213-229, 421-430)
//   min_p         drop weights below min_p times the best weight (231-232)
//   draw          target = u * kept mass, first candidate whose running sum exceeds it (234-242)
//   penalties     a token seen recently: positive logit / factor, negative * factor, minus
//                 presence + frequency * count; plus a per-token bias (596-616)
// What differs: no sort. The cuts are found by radix selection over an order-preserving integer
// key of the logit, masses are summed as 2^-40 fixed-point integers (so every sum is exact and has
// no order), and the draw walks the kept tokens in id order. The kept set is the reference's up to
// rounding at a cut's edge; which kept token a given u selects differs, the distribution does not.
#include "common.h"

namespace {
constexpr int THREADS = 1024;
constexpr int WAVES = THREADS / WAVE;
constexpr float FIXED_ONE = 1099511627776.0f;  // 2^40

__device__ __forceinline__ bool finite_f(float v) { return (__float_as_uint(v) & 0x7f800000u) != 0x7f800000u; }

// larger float <=> larger key; finite keys are above 0x007fffff
__device__ __forceinline__ uint32_t key_of(float v) {
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, WAVE);
  return v;
}

__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  v = wave_sum_u64(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  unsigned long long total = 0;
  for (int i = 0; i < WAVES; ++i) total += scratch[i];
  return total;
}

__device__ __forceinline__ unsigned long long fixed_weight(float logit, float scale, float peak) {
  return (unsigned long long)(expf(logit * scale - peak) * FIXED_ONE);
}

struct Cut {
  uint32_t key;     // keys above it are kept
  int ties;         // of the tokens with exactly this key, the first `ties` by id are kept
};

// The best finite logit of a slice of a row (ties to the lowest id; id 0x7fffffff when none is finite): grid
// (slices, rows). One workgroup per row reads a 152,064-column row at what one CU can pull (25 us); thirty-two
// slices a row spread it over the GPU, and sample_kernel then compares the slices' winners.
__global__ __launch_bounds__(256) void argmax_slices_kernel(const float* __restrict__ logits, int vocab, int slice_len,
                                                            float* __restrict__ slice_best, int* __restrict__ slice_id) {
  __shared__ float red_f[4];
  __shared__ int red_i[4];
  const int row = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* x = logits + (size_t)row * vocab;
  const int begin = blockIdx.x * slice_len, end = min(vocab, begin + slice_len);
  float b4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
  int i4[4] = {0x7fffffff, 0x7fffffff, 0x7fffffff, 0x7fffffff};
  for (int base = begin + tid; base < end; base += 4 * 256) {
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const int i = base + u * 256;
      const float v = i < end ? x[i] : NAN;
      if (finite_f(v) && v > b4[u]) {  // within one candidate the indices ascend, so ties keep the lower one
        b4[u] = v;
        i4[u] = i;
      }
    }
  }
  float best = -INFINITY;
  int best_id = 0x7fffffff;
#pragma unroll
  for (int u = 0; u < 4; ++u)
    if (b4[u] > best || (b4[u] == best && i4[u] < best_id)) {
      best = b4[u];
      best_id = i4[u];
    }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, 64);
    const int oi = __shfl_xor(best_id, off, 64);
    if (ov > best || (ov == best && oi < best_id)) {
      best = ov;
      best_id = oi;
    }
  }
  if (lane == 0) {
    red_f[wave] = best;
    red_i[wave] = best_id;
  }
  __syncthreads();
  if (tid == 0) {
    for (int w = 1; w < 4; ++w)
      if (red_f[w] > best || (red_f[w] == best && red_i[w] < best_id)) {
        best = red_f[w];
        best_id = red_i[w];
      }
    slice_best[(size_t)row * gridDim.x + blockIdx.x] = best;
    slice_id[(size_t)row * gridDim.x + blockIdx.x] = best_id;
  }
}

// Where a row's uniform comes from when it is not handed in: the request's record in the table of state slots,
// two 64-bit words per slot: the state of its xorshift64* generator (crates/vipera-sampler/src/rng.rs:13-57:
// x ^= x >> 12, x ^= x << 25, x ^= x >> 27, output x * 0x2545F4914F6CDD1D, top 53 bits as a double in [0, 1))
// and the position of the request's next token. A row that draws advances its generator by one step; a
// greedy row leaves it alone; `reseed` puts `seed_state` into the slot first (a request's first row in a slot).
struct SlotRows {
  const int* slot;                         // per row
  const int* position;                     // per row: where the token drawn now will sit
  const int* reseed;                       // per row: 0 or 1
  const unsigned long long* seed_state;    // per row
  unsigned long long* table;               // [num_slots, 2], or nullptr: the uniforms are handed in
  int num_slots;
};

// One row. Returns the chosen token in *out (or -1 when no logit is finite). `slices` > 0: the row's best logit
// comes from the winners that argmax_slices_kernel left.
__global__ __launch_bounds__(THREADS) void sample_kernel(const float* __restrict__ logits, int vocab,
                                                         const float* __restrict__ temperature,
                                                         const int* __restrict__ top_k,
                                                         const float* __restrict__ top_p,
                                                         const float* __restrict__ min_p,
                                                         const double* __restrict__ uniform, int* __restrict__ out,
                                                         const float* __restrict__ slice_best,
                                                         const int* __restrict__ slice_id, int slices, SlotRows slots) {
  __shared__ float red_f[16];
  __shared__ int red_i[WAVES];
  __shared__ unsigned long long red_u[WAVES];
  __shared__ unsigned long long hist[256];
  __shared__ uint32_t sh_key;
  __shared__ long long sh_remaining;
  __shared__ unsigned long long sh_below;

  __shared__ double sh_uniform;

  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const float* x = logits + (size_t)row * vocab;
  if (tid == 0) {
    double u = uniform ? uniform[row] : 0.0;
    const int slot = slots.table ? slots.slot[row] : -1;
    if (slot >= 0 && slot < slots.num_slots) {
      unsigned long long* record = slots.table + 2 * (size_t)slot;
      unsigned long long state = slots.reseed[row] ? slots.seed_state[row] : record[0];
      if (temperature[row] > 0.f) {
        state ^= state >> 12;
        state ^= state << 25;
        state ^= state >> 27;
        u = (double)((state * 0x2545F4914F6CDD1Dull) >> 11) * (1.0 / 9007199254740992.0);
      }
      record[0] = state;
      record[1] = (unsigned long long)(long long)slots.position[row];
    }
    sh_uniform = u;   // read after the barriers below
  }

  // --- best finite logit, ties to the lowest id ----------------------------------------------
  float best = -INFINITY;
  int best_id = 0x7fffffff;
  if (slices > 0) {
    for (int s = tid; s < slices; s += THREADS) {
      const float v = slice_best[(size_t)row * slices + s];
      const int i = slice_id[(size_t)row * slices + s];
      if (i != 0x7fffffff && (v > best || (v == best && i < best_id))) {
        best = v;
        best_id = i;
      }
    }
  } else {
    // four independent candidates per thread keep four loads in flight; they are merged in index order
    float b4[4] = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};
    int i4[4] = {0x7fffffff, 0x7fffffff, 0x7fffffff, 0x7fffffff};
    for (int base = tid; base < vocab; base += 4 * THREADS) {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const int i = base + u * THREADS;
        const float v = i < vocab ? x[i] : NAN;
        if (finite_f(v) && v > b4[u]) {  // within one candidate the indices ascend, so ties keep the lower one
          b4[u] = v;
          i4[u] = i;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (b4[u] > best || (b4[u] == best && i4[u] < best_id)) {
        best = b4[u];
        best_id = i4[u];
      }
  }
#pragma unroll
  for (int off = WAVE / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(best, off, WAVE);
    const int oi = __shfl_xor(best_id, off, WAVE);
    if (ov > best || (ov == best && oi < best_id)) {
      best = ov;
      best_id = oi;
    }
  }
  if (lane == 0) {
    red_f[wave] = best;
    red_i[wave] = best_id;
  }
  __syncthreads();
  best = red_f[0];
  best_id = red_i[0];
  for (int w = 1; w < WAVES; ++w)
    if (red_f[w] > best || (red_f[w] == best && red_i[w] < best_id)) {
      best = red_f[w];
      best_id = red_i[w];
    }
  __syncthreads();
  if (best_id == 0x7fffffff) {
    if (tid == 0) out[row] = -1;
    return;
  }
  const float temp = temperature[row];
  if (!(temp > 0.f)) {
    if (tid == 0) out[row] = best_id;
    return;
  }
  const float scale = 1.0f / temp;
  const float peak = best * scale;

  // --- top-k: the key of the k-th best token and how many of its ties are inside --------------
  Cut cut = {0u, 0x7fffffff};  // everything finite
  const int k = top_k[row];
  int finite_count = 0;
  for (int i = tid; i < vocab; i += THREADS) finite_count += finite_f(x[i]) ? 1 : 0;
  finite_count = (int)block_sum_u64((unsigned long long)finite_count, red_u);
  if (k > 0 && k < finite_count) {
    uint32_t prefix = 0;
    long long remaining = k;  // the k-th best lies among the keys that match the prefix
    for (int shift = 24; shift >= 0; shift -= 8) {
      for (int b = tid; b < 256; b += THREADS) hist[b] = 0;
      __syncthreads();
      const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
      for (int i = tid; i < vocab; i += THREADS) {
        const float v = x[i];
        if (!finite_f(v)) continue;
        const uint32_t key = key_of(v);
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1ull);
      }
      __syncthreads();
      if (tid == 0) {
        long long left = remaining;
        int b = 255;
        for (; b > 0; --b) {
          if ((long long)hist[b] >= left) break;
          left -= (long long)hist[b];
        }
        sh_key = prefix | ((uint32_t)b << shift);
        sh_remaining = left;
      }
      __syncthreads();
      prefix = sh_key;
      remaining = sh_remaining;
      __syncthreads();
    }
    cut.key = prefix;
    cut.ties = (int)remaining;
  }

  // --- top-p: the shortest head of the top-k set whose mass reaches top_p * total --------------
  const float p = top_p[row];
  if (p < 1.0f) {
    unsigned long long total = 0;
    for (int i = tid; i < vocab; i += THREADS) {
      const float v = x[i];
      if (finite_f(v)) total += fixed_weight(v, scale, peak);
    }
    total = block_sum_u64(total, red_u);
    const unsigned long long target = (unsigned long long)((double)p * (double)total);
    // how many tokens share the top-k cut's key, and their weight: only cut.ties of them count
    int at_cut = 0;
    for (int i = tid; i < vocab; i += THREADS) {
      const float v = x[i];
      at_cut += (finite_f(v) && key_of(v) == cut.key) ? 1 : 0;
    }
    at_cut = (int)block_sum_u64((unsigned long long)at_cut, red_u);
    const int cut_excess = cut.ties < at_cut ? at_cut - cut.ties : 0;
    unsigned long long cut_weight = 0;
    if (cut_excess > 0) {
      const uint32_t kb = cut.key;
      const float cv = __uint_as_float((kb & 0x80000000u) ? (kb & 0x7fffffffu) : ~kb);
      cut_weight = fixed_weight(cv, scale, peak);
    }
    uint32_t prefix = 0;
    unsigned long long above = 0;  // mass of keys above everything that matches the prefix
    bool reached = true;
    for (int shift = 24; shift >= 0; shift -= 8) {
      for (int b = tid; b < 256; b += THREADS) hist[b] = 0;
      __syncthreads();
      const uint32_t mask = shift == 24 ? 0u : (0xffffffffu << (shift + 8));
      for (int i = tid; i < vocab; i += THREADS) {
        const float v = x[i];
        if (!finite_f(v)) continue;
        const uint32_t key = key_of(v);
        if (key < cut.key) continue;  // outside the top-k set
        if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], fixed_weight(v, scale, peak));
      }
      __syncthreads();
      if (tid == 0) {
        if (cut_excess > 0 && (cut.key & mask) == prefix)
          hist[(cut.key >> shift) & 255u] -= (unsigned long long)cut_excess * cut_weight;
        unsigned long long running = above;
        int b = 255;
        bool found = false;
        for (; b >= 0; --b) {
          if (running + hist[b] >= target) {
            found = true;
            break;
          }
          running += hist[b];
        }
        if (!found) b = 0;
        sh_key = prefix | ((uint32_t)b << shift);
        sh_below = running;
        sh_remaining = found ? 1 : 0;
      }
      __syncthreads();
      prefix = sh_key;
      above = sh_below;
      reached = sh_remaining != 0;
      __syncthreads();
      if (!reached) break;
    }
    if (reached && prefix >= cut.key) {
      // tokens with key == prefix all weigh the same; take as many as the target still needs
      const float cv = __uint_as_float((prefix & 0x80000000u) ? (prefix & 0x7fffffffu) : ~prefix);
      const unsigned long long w = fixed_weight(cv, scale, peak);
      long long need = 1;
      if (w > 0 && target > above) need = (long long)((target - above + w - 1) / w);
      if (need < 1) need = 1;
      int limit = 0x7fffffff;
      if (prefix == cut.key) limit = cut.ties;
      cut.key = prefix;
      cut.ties = need < (long long)limit ? (int)need : limit;
    }
  }
  const float floor_weight = min_p[row];  // the best weight is exp(0) = 1

  // --- draw among the kept tokens in id order ------------------------------------------------------
  // every wave owns a contiguous range of ids and walks it in runs of 64
  const int span = ((vocab + WAVES - 1) / WAVES + WAVE - 1) / WAVE * WAVE;
  const int begin = wave * span, end = min(vocab, begin + span);

  // ties at the cut: rank base of every wave
  int ties_here = 0;
  for (int base = begin; base < end; base += WAVE) {
    const int i = base + lane;
    const float v = i < end ? x[i] : NAN;
    ties_here += (finite_f(v) && key_of(v) == cut.key) ? 1 : 0;
  }
  ties_here = (int)wave_sum_u64((unsigned long long)ties_here);
  if (lane == 0) red_i[wave] = ties_here;
  __syncthreads();
  int tie_base = 0;
  for (int w = 0; w < wave; ++w) tie_base += red_i[w];
  __syncthreads();

  // kept mass of every wave
  unsigned long long mass_here = 0;
  {
    int tie_rank = tie_base;
    for (int base = begin; base < end; base += WAVE) {
      const int i = base + lane;
      const float v = i < end ? x[i] : NAN;
      const bool fin = finite_f(v);
      const uint32_t key = fin ? key_of(v) : 0u;
      const bool tie = fin && key == cut.key;
      const unsigned long long ballot = __ballot(tie);
      const int rank = tie_rank + __popcll(ballot & ((1ull << lane) - 1ull));
      tie_rank += __popcll(ballot);
      bool kept = fin && (key > cut.key || (tie && rank < cut.ties));
      if (kept) kept = expf(v * scale - peak) >= floor_weight;
      mass_here += kept ? fixed_weight(v, scale, peak) : 0ull;
    }
  }
  mass_here = wave_sum_u64(mass_here);
  if (lane == 0) red_u[wave] = mass_here;
  __syncthreads();
  unsigned long long mass = 0, before = 0;
  for (int w = 0; w < WAVES; ++w) {
    if (w < wave) before += red_u[w];
    mass += red_u[w];
  }
  if (mass == 0) {  // every kept weight underflowed: the best token stands
    if (tid == 0) out[row] = best_id;
    return;
  }
  unsigned long long target = (unsigned long long)(sh_uniform * (double)mass);
  if (target >= mass) target = mass - 1;
  // the wave whose share holds the target walks its range once more
  if (target >= before && target < before + red_u[wave]) {
    unsigned long long running = before;
    int tie_rank = tie_base;
    for (int base = begin; base < end; base += WAVE) {
      const int i = base + lane;
      const float v = i < end ? x[i] : NAN;
      const bool fin = finite_f(v);
      const uint32_t key = fin ? key_of(v) : 0u;
      const bool tie = fin && key == cut.key;
      const unsigned long long ballot = __ballot(tie);
      const int rank = tie_rank + __popcll(ballot & ((1ull << lane) - 1ull));
      tie_rank += __popcll(ballot);
      bool kept = fin && (key > cut.key || (tie && rank < cut.ties));
      if (kept) kept = expf(v * scale - peak) >= floor_weight;
      const unsigned long long w = kept ? fixed_weight(v, scale, peak) : 0ull;
      // inclusive scan over the 64 lanes
      unsigned long long incl = w;
#pragma unroll
      for (int off = 1; off < WAVE; off <<= 1) {
        const unsigned long long other = __shfl_up(incl, off, WAVE);
        if (lane >= off) incl += other;
      }
      const bool hit = kept && target < running + incl;
      const unsigned long long hits = __ballot(hit);
      if (hits) {
        const int first = __ffsll((long long)hits) - 1;
        if (lane == first) out[row] = i;
        break;
      }
      running += __shfl(incl, WAVE - 1, WAVE);
    }
  }
}

// entries: (row, token, count) triples, unique per (row, token); applied in place
__global__ void penalize_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ rows,
                                const int* __restrict__ tokens, const int* __restrict__ counts,
                                const float* __restrict__ repetition, const float* __restrict__ presence,
                                const float* __restrict__ frequency, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int row = rows[i], token = tokens[i];
  if (token < 0 || token >= vocab) return;
  float* at = logits + (size_t)row * vocab + token;
  float v = *at;
  const float factor = repetition[row];
  if (factor != 1.0f) v = v > 0.f ? v / factor : v * factor;
  v -= presence[row] + frequency[row] * (float)counts[i];
  *at = v;
}

__global__ void bias_kernel(float* __restrict__ logits, int vocab, const int* __restrict__ rows,
                            const int* __restrict__ tokens, const float* __restrict__ values, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int token = tokens[i];
  if (token < 0 || token >= vocab) return;
  logits[(size_t)rows[i] * vocab + token] += values[i];
}
}  // namespace

// `slices` > 0 with room for num_rows * slices values in `slice_best` and `slice_id`: the rows' best logits are
// found by slices * num_rows workgroups first (worth it for a wide vocabulary); the result is the same.
//
// The uniform of a row that draws is `uniform[row]`, or with a `slot_table` ([num_slots, 2] 64-bit words; then
// `uniform` may be null) the next output of the generator in the row's slot, see SlotRows.
extern "C" int vk_sample(const float* logits, int num_rows, int vocab, const float* temperature, const int* top_k,
                         const float* top_p, const float* min_p, const double* uniform, int* out, float* slice_best,
                         int* slice_id, int slices, const int* slot, const int* position, const int* reseed,
                         const unsigned long long* seed_state, unsigned long long* slot_table, int num_slots,
                         void* stream) {
  if (num_rows <= 0) return 0;
  if (vocab <= 0 || slices < 0 || slices > 65535 || num_rows > 65535) return VK_BAD_ARGUMENT;
  if (!slot_table && !uniform) return VK_BAD_ARGUMENT;
  if (slot_table && (!slot || !position || !reseed || !seed_state || num_slots < 1)) return VK_BAD_ARGUMENT;
  const SlotRows slots{slot, position, reseed, seed_state, slot_table, num_slots};
  if (slices > 0) {
    if (!slice_best || !slice_id) return VK_BAD_ARGUMENT;
    const int slice_len = (vocab + slices - 1) / slices;
    argmax_slices_kernel<<<dim3(slices, num_rows), 256, 0, (hipStream_t)stream>>>(logits, vocab, slice_len, slice_best,
                                                                                 slice_id);
    VK_LAUNCH_CHECK();
  }
  sample_kernel<<<num_rows, THREADS, 0, (hipStream_t)stream>>>(logits, vocab, temperature, top_k, top_p, min_p,
                                                                uniform, out, slice_best, slice_id, slices, slots);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_penalize(float* logits, int vocab, const int* rows, const int* tokens, const int* counts,
                           const float* repetition, const float* presence, const float* frequency, int n,
                           void* stream) {
  if (n <= 0) return 0;
  penalize_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(logits, vocab, rows, tokens, counts, repetition,
                                                                    presence, frequency, n);
  VK_LAUNCH_CHECK();
  return 0;
}

extern "C" int vk_logit_bias(float* logits, int vocab, const int* rows, const int* tokens, const float* values, int n,
                             void* stream) {
  if (n <= 0) return 0;
  bias_kernel<<<(n + 255) / 256, 256, 0, (hipStream_t)stream>>>(logits, vocab, rows, tokens, values, n);
  VK_LAUNCH_CHECK();
  return 0;
}
