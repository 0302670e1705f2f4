// Continuous batching above the step function: admission, portions under a token budget, decoding,
// finishing, and what happens when pages run out.
//
// The reference's scheduler (crates/vipera-runtime/src/engine.rs) admits a request only if its prompt
// can fit the cache at all (396-424), moves waiting requests oldest first into the running set up to
// a bound (1125-1140), runs prompts in chunks (777-812) and ends a request at an end-of-sequence token,
// at its token budget, or when the context is full (1062-1110). It builds batches of one kind and
// alternates (683-730), and when a reservation fails it fails every request of the batch (731-741).
// Here a step mixes decode tokens and prompt portions under one token budget, and a failed
// reservation preempts instead: the most recently admitted running request gives its pages back,
// keeps its tokens, goes to the front of the waiting queue and is recomputed later.
//
// When pages run out:
//  * a decode token that finds no page preempts from the back of the running list (admission order)
//    until it has its page, or until it is the one that gives way;
//  * a prompt portion that finds no page waits while anything else moves in the step; when nothing
//    moves at all, the requests at the back give way until the oldest running request has its portion;
//  * a waiting request is admitted only while the pages of all its known tokens fit into the free
//    pages that the running requests do not still need for their known tokens, so that two long
//    prompts are not started into a pool that holds only one of them.
// Every plan moves at least one token while there is work. The request at the front of the running
// list is only ever asked to give way by itself, and then it is alone, every page is free, and its
// reservation succeeds, because `add` refuses a request that does not fit an empty pool. So the
// front request gets a token in every step unless the budget went to decode tokens, which is
// progress as well; with nothing running, every page is free and the front of the waiting queue
// passes the admission rule for the same reason. Requests end after finitely many tokens, hence
// no stall and no livelock.
#pragma once
#include <cstdint>
#include <deque>
#include <map>
#include <vector>

#include "cache_manager.h"

namespace vipera {

struct SchedulerConfig {
  int max_num_seqs;        // requests that may run at once
  int max_batched_tokens;  // tokens of one step
  int chunk_size;          // longest portion of one prompt in one step
  int max_model_len;       // longest sequence (prompt + generated)
  // 1: admit a waiting request as soon as its first portion finds pages, without leaving room for what the
  // running requests still need (more requests side by side, more recomputation when pages run out)
  int eager_admission = 0;
};

enum AddResult : int {
  ADD_OK = 0,
  ADD_EMPTY_PROMPT = 1,
  ADD_BAD_MAX_NEW = 2,
  ADD_NEVER_FITS = 3,   // the request alone needs more pages than the cache has
  ADD_TOO_LONG = 4,     // the prompt leaves no room below max_model_len
  ADD_DUPLICATE = 5,
};

enum FinishReason : int { NOT_FINISHED = 0, FINISH_STOP = 1, FINISH_LENGTH = 2 };

struct PlanEntry {
  uint64_t id;
  int start;   // position of the first token of the portion
  int count;   // tokens in the portion
  int wants_logits;  // 1 when the portion ends at the request's last known token
};

struct Plan {
  std::vector<PlanEntry> entries;
  std::vector<int> tokens;          // concatenated, in entry order
  std::vector<uint64_t> preempted;  // requests put back to waiting while this plan was made
};

class Scheduler {
 public:
  Scheduler(CacheManager* cache, SchedulerConfig config);
  AddResult add(uint64_t id, const int* tokens, int count, int max_new_tokens);
  // Decide the next step. Pages for it are reserved; `advance` must follow once the step has run.
  Plan plan();
  // The planned portion of `id` has been computed.
  void advance(uint64_t id);
  // A token was sampled for `id`. Returns why the request ended, or NOT_FINISHED.
  FinishReason append(uint64_t id, int token, bool is_end_of_sequence);
  // Overwrite the token `back` places before the request's last one (0: the last). For callers that
  // append a placeholder before the sampled token has reached the host. False when unknown or out of range.
  bool replace_token(uint64_t id, int back, int token);
  // Remove a request in any state and give back what it holds. False when unknown.
  bool cancel(uint64_t id);
  bool has_work() const { return !waiting_.empty() || !running_.empty(); }
  int num_waiting() const { return (int)waiting_.size(); }
  int num_running() const { return (int)running_.size(); }
  int preemptions() const { return preemptions_; }
  int generated_of(uint64_t id) const;
  int length_of(uint64_t id) const;

 private:
  struct Request {
    std::vector<int> tokens;  // prompt and everything generated
    int prompt_len = 0;
    int max_new = 0;
    int processed = 0;   // tokens whose keys and values are in the cache
    int planned_end = 0; // end of the portion of the plan in flight
    uint64_t admitted_at = 0;
  };
  void preempt(uint64_t id, Plan* plan);
  // Whether a request of `tokens` known tokens fits beside what the running requests still need.
  bool room_beside_running(int tokens) const;
  CacheManager* cache_;
  SchedulerConfig config_;
  std::map<uint64_t, Request> requests_;
  std::deque<uint64_t> waiting_;
  std::vector<uint64_t> running_;  // in admission order
  uint64_t admissions_ = 0;
  int preemptions_ = 0;
};

}  // namespace vipera
