// Paged cache bookkeeping: which pages of which pool a request holds.
//
// After the reference's BlockSpaceManager (csrc/include/engine/block_manager.hpp:
// 14-44, csrc/engine/block_manager.cpp:7-101): a FIFO free list, a reference
// count per page, one block table per request, everything given back at once
// when a request ends.  Added here:
//   * groups: layers with different needs (all keys, or a window of them) keep
//     pages of their own, with a pool, a page size and a block table per group;
//   * a window group gives a page back as soon as every later token is out of
//     its reach, and takes it again for another request;
//   * growth by any number of tokens (the reference grows by one token and only
//     when total % block_size == 1, block_manager.cpp:56-79);
//   * a slot of fixed-size state per live request, for mixers that carry state
//     instead of keys.
// The manager holds no device memory; it hands out page and slot numbers.
#pragma once

#include <cstdint>
#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

namespace lyp {

struct GroupSpec {
  int num_pages = 0;
  int page_size = 16;
  int window = 0;  // 0: every key is kept; W > 0: a token sees keys (pos - W, pos]
};

class CacheManager {
 public:
  CacheManager(std::vector<GroupSpec> groups, int num_state_slots);

  int num_groups() const { return static_cast<int>(groups_.size()); }
  const GroupSpec& group(int g) const { return groups_.at(g); }
  int num_free_pages(int g) const { return static_cast<int>(free_.at(g).size()); }
  int num_free_slots() const { return static_cast<int>(free_slots_.size()); }
  int num_state_slots() const { return num_state_slots_; }
  int num_requests() const { return static_cast<int>(requests_.size()); }

  bool has(int64_t id) const { return requests_.count(id) != 0; }

  // Registers a request and gives it a state slot.  Throws if the id is live or
  // no slot is free.
  int add(int64_t id);

  // Tokens whose keys the request holds (what commit() last said).
  int length(int64_t id) const;
  // Tokens the request's pages can hold (what extend() last said).
  int capacity(int64_t id) const;

  // Pages that growing to new_len tokens would take from group g.  An unknown
  // id counts as an empty request.
  int pages_needed(int64_t id, int g, int new_len) const;
  // Most pages of group g that a request of `len` tokens holds at one time when
  // it is computed in portions of at most `portion` tokens.
  int pages_held_at_most(int g, int len, int portion) const;
  // Longest the request can become with the pages that are free now.
  int max_length(int64_t id) const;
  // True if every group has the pages, and, for an unknown id, a slot is free.
  bool can_extend(int64_t id, int new_len) const;
  // Takes the pages for positions < new_len.  Throws, and changes nothing, if a
  // group runs out.
  void extend(int64_t id, int new_len);
  // The step that computed positions < new_len is done: window groups give
  // back the pages no later token can see.
  void commit(int64_t id, int new_len);
  // Gives everything back.  Unknown ids are ignored
  // (csrc/engine/block_manager.cpp:83-86).
  void free(int64_t id);
  void reset();

  // Logical page -> physical page, -1 where a window group gave the page back.
  const std::vector<int32_t>& table(int64_t id, int g) const;
  int state_slot(int64_t id) const;
  int ref_count(int g, int page) const { return ref_.at(g).at(page); }

  // Walks every structure and returns a description of the first broken
  // invariant (a page lost, held twice, free and held, a count that is off), or
  // an empty string.
  std::string check() const;

  struct Counters {
    int64_t pages_taken = 0, pages_returned = 0, window_returns = 0;
    int high_water = 0;  // most pages in use at once, over all groups
  };
  const Counters& counters() const { return counters_; }

 private:
  struct Request {
    int length = 0;
    int capacity = 0;
    int slot = -1;
    std::vector<std::vector<int32_t>> tables;  // per group
  };

  void release_page(int g, int32_t page);
  void note_usage();

  std::vector<GroupSpec> groups_;
  int num_state_slots_;
  std::vector<std::deque<int32_t>> free_;
  std::vector<std::vector<int32_t>> ref_;
  std::deque<int32_t> free_slots_;
  std::unordered_map<int64_t, Request> requests_;
  Counters counters_;
};

}  // namespace lyp
