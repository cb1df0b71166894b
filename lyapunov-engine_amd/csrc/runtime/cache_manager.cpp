#include "cache_manager.hpp"

#include <algorithm>
#include <climits>
#include <sstream>
#include <stdexcept>

namespace lyp {

namespace {
int ceil_div(int a, int b) { return (a + b - 1) / b; }
}  // namespace

CacheManager::CacheManager(std::vector<GroupSpec> groups, int num_state_slots)
    : groups_(std::move(groups)), num_state_slots_(num_state_slots) {
  if (groups_.empty()) throw std::invalid_argument("cache manager needs at least one group");
  for (const auto& g : groups_) {
    if (g.num_pages <= 0 || g.page_size <= 0 || g.window < 0)
      throw std::invalid_argument("cache group needs num_pages > 0, page_size > 0, window >= 0");
  }
  if (num_state_slots_ <= 0) throw std::invalid_argument("cache manager needs at least one state slot");
  reset();
}

void CacheManager::reset() {
  free_.assign(groups_.size(), {});
  ref_.assign(groups_.size(), {});
  for (size_t g = 0; g < groups_.size(); ++g) {
    ref_[g].assign(groups_[g].num_pages, 0);
    for (int p = 0; p < groups_[g].num_pages; ++p) free_[g].push_back(p);
  }
  free_slots_.clear();
  for (int s = 0; s < num_state_slots_; ++s) free_slots_.push_back(s);
  requests_.clear();
}

int CacheManager::add(int64_t id) {
  if (has(id)) throw std::runtime_error("request " + std::to_string(id) + " is already live");
  if (free_slots_.empty()) throw std::runtime_error("no free state slot");
  Request r;
  r.slot = free_slots_.front();
  free_slots_.pop_front();
  r.tables.assign(groups_.size(), {});
  requests_.emplace(id, std::move(r));
  return requests_.at(id).slot;
}

int CacheManager::length(int64_t id) const { return requests_.at(id).length; }
int CacheManager::capacity(int64_t id) const { return requests_.at(id).capacity; }

int CacheManager::pages_needed(int64_t id, int g, int new_len) const {
  const int want = ceil_div(new_len, groups_.at(g).page_size);
  auto it = requests_.find(id);
  const int have = it == requests_.end() ? 0 : static_cast<int>(it->second.tables[g].size());
  return std::max(0, want - have);
}

int CacheManager::pages_held_at_most(int g, int len, int portion) const {
  const GroupSpec& spec = groups_.at(g);
  const int all = ceil_div(len, spec.page_size);
  if (spec.window <= 0) return all;
  return std::min(all, ceil_div(spec.window + std::max(portion, 1), spec.page_size) + 1);
}

int CacheManager::max_length(int64_t id) const {
  auto it = requests_.find(id);
  if (it == requests_.end() && free_slots_.empty()) return 0;
  int64_t best = INT32_MAX;
  for (int g = 0; g < num_groups(); ++g) {
    const int64_t have = it == requests_.end() ? 0 : static_cast<int64_t>(it->second.tables[g].size());
    best = std::min<int64_t>(best, (have + num_free_pages(g)) * groups_[g].page_size);
  }
  return static_cast<int>(best);
}

bool CacheManager::can_extend(int64_t id, int new_len) const {
  if (!has(id) && free_slots_.empty()) return false;
  for (int g = 0; g < num_groups(); ++g)
    if (pages_needed(id, g, new_len) > num_free_pages(g)) return false;
  return true;
}

void CacheManager::extend(int64_t id, int new_len) {
  Request& r = requests_.at(id);
  if (new_len < r.length) throw std::runtime_error("a request cannot shrink");
  for (int g = 0; g < num_groups(); ++g) {
    if (pages_needed(id, g, new_len) > num_free_pages(g))
      throw std::runtime_error("out of pages in cache group " + std::to_string(g));
  }
  for (int g = 0; g < num_groups(); ++g) {
    const int n = pages_needed(id, g, new_len);
    for (int i = 0; i < n; ++i) {
      const int32_t page = free_[g].front();
      free_[g].pop_front();
      ref_[g][page] = 1;
      r.tables[g].push_back(page);
      ++counters_.pages_taken;
    }
  }
  r.capacity = std::max(r.capacity, new_len);
  note_usage();
}

void CacheManager::release_page(int g, int32_t page) {
  if (--ref_[g][page] <= 0) {
    ref_[g][page] = 0;
    free_[g].push_back(page);
    ++counters_.pages_returned;
  }
}

void CacheManager::commit(int64_t id, int new_len) {
  Request& r = requests_.at(id);
  if (new_len > r.capacity) throw std::runtime_error("commit beyond the pages the request holds");
  if (new_len < r.length) throw std::runtime_error("a request cannot shrink");
  r.length = new_len;
  for (int g = 0; g < num_groups(); ++g) {
    const GroupSpec& spec = groups_[g];
    if (spec.window <= 0) continue;
    // The next token sits at position new_len and sees keys > new_len - window.
    const int first_needed = new_len - spec.window + 1;
    auto& table = r.tables[g];
    for (size_t i = 0; i < table.size(); ++i) {
      if (static_cast<int>(i + 1) * spec.page_size > first_needed) break;
      if (table[i] >= 0) {
        release_page(g, table[i]);
        table[i] = -1;
        ++counters_.window_returns;
      }
    }
  }
}

void CacheManager::free(int64_t id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return;
  for (int g = 0; g < num_groups(); ++g)
    for (int32_t page : it->second.tables[g])
      if (page >= 0) release_page(g, page);
  free_slots_.push_back(it->second.slot);
  requests_.erase(it);
}

const std::vector<int32_t>& CacheManager::table(int64_t id, int g) const { return requests_.at(id).tables.at(g); }
int CacheManager::state_slot(int64_t id) const { return requests_.at(id).slot; }

void CacheManager::note_usage() {
  int used = 0;
  for (int g = 0; g < num_groups(); ++g) used += groups_[g].num_pages - num_free_pages(g);
  counters_.high_water = std::max(counters_.high_water, used);
}

std::string CacheManager::check() const {
  std::ostringstream err;
  for (int g = 0; g < num_groups(); ++g) {
    const int n = groups_[g].num_pages;
    std::vector<int> held(n, 0), in_free(n, 0);
    for (int32_t p : free_[g]) {
      if (p < 0 || p >= n) return "group " + std::to_string(g) + ": free list holds page " + std::to_string(p);
      if (++in_free[p] > 1) return "group " + std::to_string(g) + ": page " + std::to_string(p) + " is free twice";
    }
    for (const auto& [id, r] : requests_) {
      for (int32_t p : r.tables[g]) {
        if (p < 0) continue;
        if (p >= n) return "request " + std::to_string(id) + " holds page " + std::to_string(p) + " out of range";
        ++held[p];
      }
    }
    for (int p = 0; p < n; ++p) {
      if (held[p] != ref_[g][p]) {
        err << "group " << g << ": page " << p << " is in " << held[p] << " tables but counted " << ref_[g][p];
        return err.str();
      }
      if (held[p] > 0 && in_free[p]) {
        err << "group " << g << ": page " << p << " is held and free";
        return err.str();
      }
      if (held[p] == 0 && !in_free[p]) {
        err << "group " << g << ": page " << p << " is lost";
        return err.str();
      }
      if (held[p] > 1) {
        err << "group " << g << ": page " << p << " is held " << held[p] << " times";
        return err.str();
      }
    }
  }
  std::vector<int> slot_use(num_state_slots_, 0);
  for (int s : free_slots_) {
    if (s < 0 || s >= num_state_slots_ || ++slot_use[s] > 1) return "state slot " + std::to_string(s) + " is free twice";
  }
  for (const auto& [id, r] : requests_) {
    if (r.slot < 0 || r.slot >= num_state_slots_ || ++slot_use[r.slot] > 1)
      return "state slot " + std::to_string(r.slot) + " of request " + std::to_string(id) + " is shared or free";
    if (r.length > r.capacity) return "request " + std::to_string(id) + " is longer than its pages";
    for (int g = 0; g < num_groups(); ++g) {
      const int pages = static_cast<int>(r.tables[g].size());
      if (pages * groups_[g].page_size < r.capacity) return "request " + std::to_string(id) + " lacks pages for its capacity";
    }
  }
  for (int s = 0; s < num_state_slots_; ++s)
    if (slot_use[s] != 1) return "state slot " + std::to_string(s) + " is lost";
  return "";
}

}  // namespace lyp
