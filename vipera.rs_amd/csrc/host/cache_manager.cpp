#include "cache_manager.h"

#include <algorithm>
#include <sstream>

namespace vipera {

BlockPool::BlockPool(int num_blocks) : total_(num_blocks), held_(num_blocks > 0 ? num_blocks : 0, 0) {
  free_.reserve(held_.size());
  // reversed, so that taking from the back hands out the lowest id first
  for (int id = num_blocks - 1; id >= 0; --id) free_.push_back(id);
}

int BlockPool::take() {
  if (free_.empty()) return -1;
  const int id = free_.back();
  free_.pop_back();
  held_[id] = 1;
  return id;
}

bool BlockPool::give_back(int id) {
  if (id < 0 || id >= total_ || !held_[id]) return false;
  held_[id] = 0;
  free_.push_back(id);
  return true;
}

CacheManager::CacheManager(std::vector<GroupConfig> groups, int num_slots)
    : groups_(std::move(groups)), num_slots_(num_slots) {
  for (const auto& g : groups_) pools_.emplace_back(g.num_blocks);
  for (int s = num_slots - 1; s >= 0; --s) free_slots_.push_back(s);
}

int CacheManager::first_block_needed(int g, int start) const {
  const GroupConfig& cfg = groups_[g];
  if (cfg.window <= 0) return 0;
  const int lo = std::max(0, start + 1 - cfg.window);  // first position visible to the token at `start`
  return lo / cfg.block_size;
}

int CacheManager::blocks_needed(int g, int total, int portion) const {
  const GroupConfig& cfg = groups_[g];
  const int all = (total + cfg.block_size - 1) / cfg.block_size;
  if (cfg.window <= 0) return all;
  // a portion [s, s + portion) holds positions [s + 1 - window, s + portion): at most
  // window - 1 + portion positions, which touch at most that many / block_size + 1 pages
  const int span = cfg.window - 1 + std::max(1, portion);
  return std::min(all, span / cfg.block_size + 2);
}

ReserveResult CacheManager::reserve(uint64_t id, int start, int total) {
  Timed timed(&allocate_nanos_);
  if (start < 0) start = 0;
  if (total < start) total = start;
  auto found = requests_.find(id);
  const bool is_new = found == requests_.end();
  // first pass: count what is missing
  std::vector<int> first(groups_.size()), last(groups_.size()), missing(groups_.size(), 0);
  for (size_t g = 0; g < groups_.size(); ++g) {
    first[g] = first_block_needed((int)g, start);
    last[g] = (total + groups_[g].block_size - 1) / groups_[g].block_size;  // exclusive
    int need = 0, need_at_once = 0;
    for (int b = first[g]; b < last[g]; ++b) {
      const bool have = !is_new && b < (int)found->second.tables[g].size() && found->second.tables[g][b] >= 0;
      if (!have) ++need;
      ++need_at_once;
    }
    if (need_at_once > pools_[g].total()) return RESERVE_NEVER_FITS;
    missing[g] = need;
    if (need > pools_[g].free_count()) return RESERVE_NO_PAGES;
  }
  if (is_new && free_slots_.empty()) return RESERVE_NO_SLOT;
  // second pass: take
  if (is_new) {
    Held held;
    held.slot = free_slots_.back();
    free_slots_.pop_back();
    held.tables.resize(groups_.size());
    found = requests_.emplace(id, std::move(held)).first;
  }
  for (size_t g = 0; g < groups_.size(); ++g) {
    auto& table = found->second.tables[g];
    if ((int)table.size() < last[g]) table.resize(last[g], -1);
    for (int b = first[g]; b < last[g]; ++b)
      if (table[b] < 0) table[b] = pools_[g].take();
  }
  return RESERVE_OK;
}

void CacheManager::advance(uint64_t id, int processed) {
  Timed timed(&allocate_nanos_);
  auto found = requests_.find(id);
  if (found == requests_.end()) return;
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g].window <= 0) continue;
    auto& table = found->second.tables[g];
    const int keep_from = std::min(first_block_needed((int)g, processed), (int)table.size());
    for (int b = 0; b < keep_from; ++b) {
      if (table[b] >= 0) {
        if (!pools_[g].give_back(table[b])) ++bad_frees_;
        table[b] = -1;
      }
    }
  }
}

bool CacheManager::release(uint64_t id) {
  Timed timed(&allocate_nanos_);
  auto found = requests_.find(id);
  if (found == requests_.end()) return false;
  for (size_t g = 0; g < groups_.size(); ++g) {
    auto& table = found->second.tables[g];
    // highest block first, so the request's first page is the next one handed out
    for (int b = (int)table.size() - 1; b >= 0; --b)
      if (table[b] >= 0 && !pools_[g].give_back(table[b])) ++bad_frees_;
  }
  free_slots_.push_back(found->second.slot);
  requests_.erase(found);
  return true;
}

const std::vector<int>& CacheManager::table(uint64_t id, int group) const {
  auto found = requests_.find(id);
  if (found == requests_.end() || group < 0 || group >= (int)groups_.size()) return empty_;
  return found->second.tables[group];
}

int CacheManager::slot(uint64_t id) const {
  auto found = requests_.find(id);
  return found == requests_.end() ? -1 : found->second.slot;
}

int CacheManager::held_blocks(uint64_t id, int g) const {
  int held = 0;
  for (int page : table(id, g)) held += page >= 0;
  return held;
}

std::string CacheManager::check() const {
  std::ostringstream problem;
  if (bad_frees_) problem << bad_frees_ << " pages were freed while not held; ";
  for (size_t g = 0; g < groups_.size(); ++g) {
    std::vector<int> owners(pools_[g].total(), 0);
    for (const auto& [id, held] : requests_) {
      for (int page : held.tables[g]) {
        if (page < 0) continue;
        if (page >= pools_[g].total()) {
          problem << "group " << g << ": request " << id << " holds page " << page << " outside the pool; ";
          continue;
        }
        ++owners[page];
      }
    }
    int held_count = 0;
    for (int page = 0; page < pools_[g].total(); ++page) {
      if (owners[page] > 1) problem << "group " << g << ": page " << page << " is held " << owners[page] << " times; ";
      if (owners[page] == 1 && !pools_[g].is_held(page))
        problem << "group " << g << ": page " << page << " is in a table but marked free; ";
      if (owners[page] == 0 && pools_[g].is_held(page))
        problem << "group " << g << ": page " << page << " is lost (held by nobody, not free); ";
      held_count += owners[page] > 0;
    }
    if (held_count + pools_[g].free_count() != pools_[g].total())
      problem << "group " << g << ": " << held_count << " held + " << pools_[g].free_count() << " free != "
              << pools_[g].total() << "; ";
  }
  std::vector<int> slot_owners(num_slots_, 0);
  for (const auto& [id, held] : requests_) {
    if (held.slot < 0 || held.slot >= num_slots_)
      problem << "request " << id << " has slot " << held.slot << "; ";
    else
      ++slot_owners[held.slot];
  }
  for (int s : free_slots_)
    if (s >= 0 && s < num_slots_) ++slot_owners[s];
  for (int s = 0; s < num_slots_; ++s)
    if (slot_owners[s] != 1) problem << "slot " << s << " is accounted for " << slot_owners[s] << " times; ";
  return problem.str();
}

}  // namespace vipera
