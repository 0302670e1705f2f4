// C interface of the host library, for ctypes. Handles are opaque pointers; functions return
// status codes or counts and never throw across the boundary.
#include <cstring>
#include <new>
#include <string>

#include "cache_manager.h"
#include "scheduler.h"

using namespace vipera;

namespace {
struct SchedulerHandle {
  Scheduler scheduler;
  Plan plan;
  SchedulerHandle(CacheManager* cache, SchedulerConfig config) : scheduler(cache, config) {}
};
}  // namespace

extern "C" {

void* vk_cache_create(int num_groups, const int* block_sizes, const int* num_blocks, const int* windows,
                      int num_slots) {
  if (num_groups < 0 || num_slots < 0) return nullptr;
  std::vector<GroupConfig> groups;
  for (int g = 0; g < num_groups; ++g) {
    if (block_sizes[g] <= 0 || num_blocks[g] < 0 || windows[g] < 0) return nullptr;
    groups.push_back({block_sizes[g], num_blocks[g], windows[g]});
  }
  return new (std::nothrow) CacheManager(std::move(groups), num_slots);
}

void vk_cache_destroy(void* handle) { delete static_cast<CacheManager*>(handle); }

int vk_cache_reserve(void* handle, unsigned long long id, int start, int total) {
  return static_cast<CacheManager*>(handle)->reserve(id, start, total);
}

void vk_cache_advance(void* handle, unsigned long long id, int processed) {
  static_cast<CacheManager*>(handle)->advance(id, processed);
}

int vk_cache_release(void* handle, unsigned long long id) {
  return static_cast<CacheManager*>(handle)->release(id) ? 0 : 1;
}

// Copies the block table (page per logical block, -1 for none) into `out`; returns its length,
// which may exceed `capacity` (then only `capacity` entries were written).
int vk_cache_table(void* handle, unsigned long long id, int group, int* out, int capacity) {
  const auto& table = static_cast<CacheManager*>(handle)->table(id, group);
  const int n = (int)table.size();
  if (out && capacity > 0) std::memcpy(out, table.data(), sizeof(int) * (size_t)(n < capacity ? n : capacity));
  return n;
}

// The block tables of `count` requests at once: row k of out[count][width] gets the table of ids[k]
// (-1 where it holds no page, and past its end). Logical blocks [from[k], to[k]) of request k must all
// be backed by a page and fit the row. Returns -1 when that holds for every request, else the index of
// the first one for which it does not (rows up to that one are written).
int vk_cache_fill_tables(void* handle, const unsigned long long* ids, int count, int group, int* out, int width,
                         const int* from, const int* to) {
  const CacheManager* cache = static_cast<CacheManager*>(handle);
  for (int k = 0; k < count; ++k) {
    const auto& table = cache->table(ids[k], group);
    const int n = (int)table.size() < width ? (int)table.size() : width;
    int* row = out + (size_t)k * width;
    if (n > 0) std::memcpy(row, table.data(), sizeof(int) * (size_t)n);
    for (int b = n; b < width; ++b) row[b] = -1;
    if (to[k] > n) return k;
    for (int b = from[k] < 0 ? 0 : from[k]; b < to[k]; ++b)
      if (row[b] < 0) return k;
  }
  return -1;
}

unsigned long long vk_cache_allocate_nanos(void* handle) { return static_cast<CacheManager*>(handle)->allocate_nanos(); }

int vk_cache_slot(void* handle, unsigned long long id) { return static_cast<CacheManager*>(handle)->slot(id); }
int vk_cache_knows(void* handle, unsigned long long id) { return static_cast<CacheManager*>(handle)->knows(id) ? 1 : 0; }
int vk_cache_free_blocks(void* handle, int group) { return static_cast<CacheManager*>(handle)->free_blocks(group); }
int vk_cache_used_blocks(void* handle, int group) { return static_cast<CacheManager*>(handle)->used_blocks(group); }
int vk_cache_free_slots(void* handle) { return static_cast<CacheManager*>(handle)->free_slots(); }
int vk_cache_live_requests(void* handle) { return static_cast<CacheManager*>(handle)->live_requests(); }
int vk_cache_blocks_needed(void* handle, int group, int total, int portion) {
  return static_cast<CacheManager*>(handle)->blocks_needed(group, total, portion);
}

// Writes a description of what is wrong (empty when nothing is) into `out`; returns its length.
int vk_cache_check(void* handle, char* out, int capacity) {
  const std::string text = static_cast<CacheManager*>(handle)->check();
  if (out && capacity > 0) {
    const size_t n = text.size() < (size_t)capacity - 1 ? text.size() : (size_t)capacity - 1;
    std::memcpy(out, text.data(), n);
    out[n] = 0;
  }
  return (int)text.size();
}

void* vk_sched_create(void* cache, int max_num_seqs, int max_batched_tokens, int chunk_size, int max_model_len,
                      int eager_admission) {
  if (!cache) return nullptr;
  return new (std::nothrow) SchedulerHandle(
      static_cast<CacheManager*>(cache), {max_num_seqs, max_batched_tokens, chunk_size, max_model_len, eager_admission});
}

void vk_sched_destroy(void* handle) { delete static_cast<SchedulerHandle*>(handle); }

int vk_sched_add(void* handle, unsigned long long id, const int* tokens, int count, int max_new_tokens) {
  return static_cast<SchedulerHandle*>(handle)->scheduler.add(id, tokens, count, max_new_tokens);
}

// Makes the next plan and keeps it in the handle; returns the number of entries.
// `num_tokens` and `num_preempted` receive the sizes of the other two lists.
int vk_sched_plan(void* handle, int* num_tokens, int* num_preempted) {
  auto* h = static_cast<SchedulerHandle*>(handle);
  h->plan = h->scheduler.plan();
  *num_tokens = (int)h->plan.tokens.size();
  *num_preempted = (int)h->plan.preempted.size();
  return (int)h->plan.entries.size();
}

// Copies the kept plan out; every array has the size that vk_sched_plan reported.
void vk_sched_plan_read(void* handle, unsigned long long* ids, int* starts, int* counts, int* wants, int* tokens,
                        unsigned long long* preempted) {
  auto* h = static_cast<SchedulerHandle*>(handle);
  for (size_t i = 0; i < h->plan.entries.size(); ++i) {
    ids[i] = h->plan.entries[i].id;
    starts[i] = h->plan.entries[i].start;
    counts[i] = h->plan.entries[i].count;
    wants[i] = h->plan.entries[i].wants_logits;
  }
  if (!h->plan.tokens.empty()) std::memcpy(tokens, h->plan.tokens.data(), sizeof(int) * h->plan.tokens.size());
  for (size_t i = 0; i < h->plan.preempted.size(); ++i) preempted[i] = h->plan.preempted[i];
}

void vk_sched_advance(void* handle, unsigned long long id) { static_cast<SchedulerHandle*>(handle)->scheduler.advance(id); }

int vk_sched_append(void* handle, unsigned long long id, int token, int is_end_of_sequence) {
  return static_cast<SchedulerHandle*>(handle)->scheduler.append(id, token, is_end_of_sequence != 0);
}

int vk_sched_replace_token(void* handle, unsigned long long id, int back, int token) {
  return static_cast<SchedulerHandle*>(handle)->scheduler.replace_token(id, back, token) ? 0 : 1;
}

int vk_sched_cancel(void* handle, unsigned long long id) {
  return static_cast<SchedulerHandle*>(handle)->scheduler.cancel(id) ? 0 : 1;
}

int vk_sched_has_work(void* handle) { return static_cast<SchedulerHandle*>(handle)->scheduler.has_work() ? 1 : 0; }
int vk_sched_num_waiting(void* handle) { return static_cast<SchedulerHandle*>(handle)->scheduler.num_waiting(); }
int vk_sched_num_running(void* handle) { return static_cast<SchedulerHandle*>(handle)->scheduler.num_running(); }
int vk_sched_preemptions(void* handle) { return static_cast<SchedulerHandle*>(handle)->scheduler.preemptions(); }
int vk_sched_generated_of(void* handle, unsigned long long id) {
  return static_cast<SchedulerHandle*>(handle)->scheduler.generated_of(id);
}
int vk_sched_length_of(void* handle, unsigned long long id) {
  return static_cast<SchedulerHandle*>(handle)->scheduler.length_of(id);
}

}  // extern "C"
