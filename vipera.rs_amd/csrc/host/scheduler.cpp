#include "scheduler.h"

#include <algorithm>

namespace vipera {

Scheduler::Scheduler(CacheManager* cache, SchedulerConfig config) : cache_(cache), config_(config) {
  if (config_.chunk_size < 1) config_.chunk_size = 1;
  if (config_.max_batched_tokens < 1) config_.max_batched_tokens = 1;
  if (config_.max_num_seqs < 1) config_.max_num_seqs = 1;
}

AddResult Scheduler::add(uint64_t id, const int* tokens, int count, int max_new_tokens) {
  if (count <= 0) return ADD_EMPTY_PROMPT;
  if (max_new_tokens < 1) return ADD_BAD_MAX_NEW;
  if (requests_.count(id)) return ADD_DUPLICATE;
  if (count + 1 > config_.max_model_len) return ADD_TOO_LONG;
  // the longest the request can get: every token but the last one sampled is fed back
  const int longest = std::min(config_.max_model_len, count + max_new_tokens - 1);
  const int portion = std::min(config_.chunk_size, config_.max_batched_tokens);
  for (int g = 0; g < cache_->num_groups(); ++g)
    if (cache_->blocks_needed(g, longest, portion) > cache_->group(g).num_blocks) return ADD_NEVER_FITS;
  Request request;
  request.tokens.assign(tokens, tokens + count);
  request.prompt_len = count;
  request.max_new = max_new_tokens;
  requests_.emplace(id, std::move(request));
  waiting_.push_back(id);
  return ADD_OK;
}

void Scheduler::preempt(uint64_t id, Plan* plan) {
  cache_->release(id);
  Request& request = requests_[id];
  request.processed = 0;
  request.planned_end = 0;
  running_.erase(std::remove(running_.begin(), running_.end(), id), running_.end());
  waiting_.push_front(id);
  ++preemptions_;
  // a request preempted after its portion was planned leaves the plan again
  auto& entries = plan->entries;
  entries.erase(std::remove_if(entries.begin(), entries.end(), [id](const PlanEntry& e) { return e.id == id; }),
                entries.end());
  plan->preempted.push_back(id);
}

bool Scheduler::room_beside_running(int tokens) const {
  const int portion = std::min(config_.chunk_size, config_.max_batched_tokens);
  for (int g = 0; g < cache_->num_groups(); ++g) {
    long spoken_for = 0;
    for (uint64_t id : running_) {
      const Request& request = requests_.at(id);
      const int need = cache_->blocks_needed(g, (int)request.tokens.size(), portion);
      spoken_for += std::max(0, need - cache_->held_blocks(id, g));
    }
    if (cache_->free_blocks(g) - spoken_for < cache_->blocks_needed(g, tokens, portion)) return false;
  }
  return true;
}

Plan Scheduler::plan() {
  Plan plan;
  int budget = config_.max_batched_tokens;

  // 1. every running request that waits for one token (decoding) gets it; when a page is missing the
  //    most recently admitted running request gives way
  std::vector<uint64_t> order = running_;
  for (uint64_t id : order) {
    if (std::find(running_.begin(), running_.end(), id) == running_.end()) continue;  // preempted meanwhile
    Request& request = requests_[id];
    const int remaining = (int)request.tokens.size() - request.processed;
    if (remaining != 1 || request.processed == 0) continue;
    if (budget < 1) break;
    for (;;) {
      const ReserveResult result = cache_->reserve(id, request.processed, request.processed + 1);
      if (result == RESERVE_OK) {
        plan.entries.push_back({id, request.processed, 1, 1});
        request.planned_end = request.processed + 1;
        --budget;
        break;
      }
      const uint64_t victim = running_.back();
      preempt(victim, &plan);
      if (victim == id) break;
      // the victim may have held a planned decode token of this step: its budget comes back
      budget = config_.max_batched_tokens - (int)plan.entries.size();
    }
  }

  // 2. running requests in the middle of a prompt (or recomputing after a preemption); a portion that
  //    finds no page waits as long as anything else moves in this step
  for (uint64_t id : running_) {
    if (budget < 1) break;
    Request& request = requests_[id];
    const int remaining = (int)request.tokens.size() - request.processed;
    if (remaining == 1 && request.processed > 0) continue;  // handled above
    if (remaining < 1) continue;
    const int count = std::min({remaining, config_.chunk_size, budget});
    if (cache_->reserve(id, request.processed, request.processed + count) != RESERVE_OK) continue;
    const int end = request.processed + count;
    plan.entries.push_back({id, request.processed, count, end == (int)request.tokens.size() ? 1 : 0});
    request.planned_end = end;
    budget -= count;
  }

  // 3. admit waiting requests, oldest first, while all they hold so far fits beside what the running
  //    requests still need for theirs
  while (!waiting_.empty() && budget >= 1 && (int)running_.size() < config_.max_num_seqs) {
    const uint64_t id = waiting_.front();
    // a request that was preempted while this plan was made waits for the next step
    if (std::find(plan.preempted.begin(), plan.preempted.end(), id) != plan.preempted.end()) break;
    Request& request = requests_[id];
    if (!config_.eager_admission && !room_beside_running((int)request.tokens.size())) break;
    const int count = std::min({(int)request.tokens.size(), config_.chunk_size, budget});
    if (cache_->reserve(id, 0, count) != RESERVE_OK) break;
    waiting_.pop_front();
    running_.push_back(id);
    request.admitted_at = ++admissions_;
    request.processed = 0;
    plan.entries.push_back({id, 0, count, count == (int)request.tokens.size() ? 1 : 0});
    request.planned_end = count;
    budget -= count;
  }

  // 4. nothing moves although requests are running: every one of them waits for a page that only
  //    another one can give back. The most recently admitted ones give way until the oldest can go on.
  //    It cannot end up giving way itself: alone it fits, or it would have been refused when added.
  if (plan.entries.empty() && !running_.empty() && budget >= 1) {
    const uint64_t id = running_.front();
    Request& request = requests_[id];
    const int remaining = (int)request.tokens.size() - request.processed;
    const int count = std::min({remaining, config_.chunk_size, budget});
    while (count >= 1) {
      if (cache_->reserve(id, request.processed, request.processed + count) == RESERVE_OK) {
        const int end = request.processed + count;
        plan.entries.push_back({id, request.processed, count, end == (int)request.tokens.size() ? 1 : 0});
        request.planned_end = end;
        budget -= count;
        break;
      }
      const uint64_t victim = running_.back();
      if (victim == id) break;
      preempt(victim, &plan);
    }
  }

  for (const PlanEntry& entry : plan.entries) {
    const Request& request = requests_[entry.id];
    plan.tokens.insert(plan.tokens.end(), request.tokens.begin() + entry.start,
                       request.tokens.begin() + entry.start + entry.count);
  }
  return plan;
}

void Scheduler::advance(uint64_t id) {
  auto found = requests_.find(id);
  if (found == requests_.end()) return;
  found->second.processed = found->second.planned_end;
  cache_->advance(id, found->second.processed);
}

FinishReason Scheduler::append(uint64_t id, int token, bool is_end_of_sequence) {
  auto found = requests_.find(id);
  if (found == requests_.end()) return NOT_FINISHED;
  Request& request = found->second;
  request.tokens.push_back(token);
  const int generated = (int)request.tokens.size() - request.prompt_len;
  FinishReason reason = NOT_FINISHED;
  if (is_end_of_sequence)
    reason = FINISH_STOP;
  else if (generated >= request.max_new)
    reason = FINISH_LENGTH;
  else if ((int)request.tokens.size() >= config_.max_model_len)
    reason = FINISH_LENGTH;  // the context is full
  if (reason != NOT_FINISHED) cancel(id);
  return reason;
}

bool Scheduler::replace_token(uint64_t id, int back, int token) {
  auto found = requests_.find(id);
  if (found == requests_.end()) return false;
  std::vector<int>& tokens = found->second.tokens;
  if (back < 0 || back >= (int)tokens.size() - found->second.prompt_len) return false;  // generated tokens only
  tokens[tokens.size() - 1 - (size_t)back] = token;
  return true;
}

bool Scheduler::cancel(uint64_t id) {
  auto found = requests_.find(id);
  if (found == requests_.end()) return false;
  cache_->release(id);
  running_.erase(std::remove(running_.begin(), running_.end(), id), running_.end());
  waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), id), waiting_.end());
  requests_.erase(found);
  return true;
}

int Scheduler::generated_of(uint64_t id) const {
  auto found = requests_.find(id);
  return found == requests_.end() ? -1 : (int)found->second.tokens.size() - found->second.prompt_len;
}

int Scheduler::length_of(uint64_t id) const {
  auto found = requests_.find(id);
  return found == requests_.end() ? -1 : (int)found->second.tokens.size();
}

}  // namespace vipera
