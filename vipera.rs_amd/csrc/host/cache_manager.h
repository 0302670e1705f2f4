// Paged cache bookkeeping on the host: page pools, per-request block tables, state slots.
//
// A *group* is a set of layers with the same needs: a page size and a retention rule (keep every
// position, or only a window of the last positions). Each group has a pool of pages of its own and
// every request has one block table per group. One page id addresses the same place in the cache
// tensors of every layer of the group. Beside the pages, a request holds one *slot*: the index of
// its fixed-size per-request state.
//
// Policy taken from the reference's cache (crates/vipera-runtime/src/kv.rs): the free list hands out
// the lowest page id first and a released page is the next one handed out (261-264, 557-559); a
// reservation is all-or-nothing, so a failed one leaves no partial table (326-382); a request that
// could never fit is told so (341-346). What differs: pages are given back when a request ends
// or when a window has moved past them, and there is no parking of finished requests.
#pragma once
#include <chrono>
#include <cstdint>
#include <map>
#include <string>
#include <vector>

namespace vipera {

struct GroupConfig {
  int block_size;  // positions per page
  int num_blocks;  // pages in the pool
  int window;      // 0: keep every position; else positions [p + 1 - window, p] are visible to p
};

class BlockPool {
 public:
  explicit BlockPool(int num_blocks);
  int free_count() const { return (int)free_.size(); }
  int total() const { return total_; }
  int take();              // lowest id first, then most recently released; -1 when empty
  bool give_back(int id);  // false when the page is not held (double free or unknown id)
  bool is_held(int id) const { return id >= 0 && id < total_ && held_[id]; }

 private:
  int total_;
  std::vector<int> free_;
  std::vector<uint8_t> held_;
};

enum ReserveResult : int {
  RESERVE_OK = 0,
  RESERVE_NO_PAGES = 1,    // not enough free pages now; nothing was changed
  RESERVE_NO_SLOT = 2,     // every state slot is taken; nothing was changed
  RESERVE_NEVER_FITS = 3,  // more pages than a pool has in total
};

class CacheManager {
 public:
  CacheManager(std::vector<GroupConfig> groups, int num_slots);

  // Make request `id` able to run tokens [start, total): afterwards every group's table maps the
  // logical blocks that positions [first visible of start, total) fall in. Tokens before `start`
  // are already in the cache. All groups or nothing.
  ReserveResult reserve(uint64_t id, int start, int total);
  // Pages of windowed groups that no position >= `processed` can see are given back.
  void advance(uint64_t id, int processed);
  // Everything the request holds is given back. False when the id is unknown.
  bool release(uint64_t id);

  bool knows(uint64_t id) const { return requests_.count(id) != 0; }
  // Block table of a request in a group: page per logical block, -1 where no page is held.
  const std::vector<int>& table(uint64_t id, int group) const;
  int slot(uint64_t id) const;
  // Pages the request holds in group g now.
  int held_blocks(uint64_t id, int g) const;
  int num_groups() const { return (int)groups_.size(); }
  const GroupConfig& group(int g) const { return groups_[g]; }
  int free_blocks(int g) const { return pools_[g].free_count(); }
  int used_blocks(int g) const { return pools_[g].total() - pools_[g].free_count(); }
  int free_slots() const { return (int)free_slots_.size(); }
  int live_requests() const { return (int)requests_.size(); }
  // Pages a request of `total` tokens needs at most at one time in group g when run in portions
  // of at most `portion` tokens.
  int blocks_needed(int g, int total, int portion) const;
  // Checks that every page is either free or held by exactly one table entry, and every slot
  // likewise. Returns an empty string when all is well, else what is wrong.
  std::string check() const;
  // Nanoseconds spent so far in reserve, advance and release: the `allocate` stage of a step's timing
  // (crates/vipera-runtime/src/pipeline.rs:251-270), whoever called them.
  uint64_t allocate_nanos() const { return allocate_nanos_; }

 private:
  struct Held {
    int slot = -1;
    std::vector<std::vector<int>> tables;  // per group
  };
  int first_block_needed(int g, int start) const;
  std::vector<GroupConfig> groups_;
  std::vector<BlockPool> pools_;
  std::vector<int> free_slots_;
  int num_slots_;
  std::map<uint64_t, Held> requests_;
  std::vector<int> empty_;
  int bad_frees_ = 0;  // pages given back that were not held: must stay 0
  uint64_t allocate_nanos_ = 0;
  struct Timed {  // adds the time of its scope to the manager's count
    uint64_t* into;
    std::chrono::steady_clock::time_point from = std::chrono::steady_clock::now();
    explicit Timed(uint64_t* total) : into(total) {}
    ~Timed() {
      *into += (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(std::chrono::steady_clock::now() - from)
                   .count();
    }
  };
};

}  // namespace vipera
