// The cache manager's bookkeeping: groups of layers with their own page allocators, a block table per
// request and group, release of pages behind a window, slots for per-request state, prefix sharing, and the
// packing of a step's batch description into one int32 buffer.  Host side only: the tensors live elsewhere.
#pragma once
#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>

#include "page_allocator.h"

namespace ta {

enum CacheStatus {
  CACHE_OK = 0, CACHE_ALREADY_LIVE = -1, CACHE_NO_SLOT = -2, CACHE_UNKNOWN_REQUEST = -3, CACHE_SHRINKS = -4,
  CACHE_TOO_FEW_PAGES = -5, CACHE_PAGE_GIVEN_BACK = -6, CACHE_TABLE_TOO_WIDE = -7, CACHE_BUFFER_TOO_SMALL = -8,
  CACHE_BAD_ARGUMENT = -9
};

// A group of layers with one need: `window` < 0 keeps the keys of every position; a window w >= 0 means that a
// query reads the keys at most w positions behind it, so pages wholly behind every later query are given back.
// (Whatever a mixer calls its kind of cache, it reaches this class as that one number.)
struct Group {
  int window;
  PageAllocator allocator;
  bool keeps_all() const { return window < 0; }
  Group(int window, int num_pages, int page_size) : window(window), allocator(num_pages, page_size) {}
};

struct Request {
  int seq_len = 0;
  int slot = -1;
  std::vector<std::vector<int>> tables;                   // per group; -1 = page given back
};

class CacheCore {
 public:
  // `n_state_layers`: how many layers keep per-request state of fixed size in the request's slot.  A prefix can
  // be shared only when what a request holds after it is a function of its pages alone: every group keeps all
  // positions and no layer keeps such state (a state slot has seen every token; an attached prefix would skip them).
  CacheCore(int n_groups, const int* windows, int num_pages, int page_size, int max_requests, bool prefix_cache,
            int n_state_layers);

  int n_groups() const { return (int)groups_.size(); }
  int page_size() const { return page_size_; }
  bool prefix_cache() const { return prefix_cache_; }
  PageAllocator* allocator(int group) { return &groups_[group]->allocator; }
  int n_requests() const { return (int)requests_.size(); }
  int free_slot_count() const { return (int)free_slots_.size(); }
  const Request* find(int64_t id) const;
  int request_ids(int64_t* out) const;

  int add_request(int64_t id);                            // the slot, or a CacheStatus
  int first_needed_position(int group, int seq_len) const;
  int pages_missing(int64_t id, int new_len, int* per_group) const;
  int can_reserve(int64_t id, int new_len) const;         // 1, 0 or a CacheStatus
  int reserve(int64_t id, int new_len);                   // 1 = done, 0 = nothing changed, or a CacheStatus
  int advance(int64_t id, int new_len);
  int release(int64_t id);
  int attach_shared_prefix(int64_t id, const int32_t* tokens, int count);   // tokens covered, or a CacheStatus
  int detach(int64_t id);
  int publish(int64_t id, const int32_t* tokens, int count);
  std::string check_invariants() const;

  // One step's batch description.  Entry i is request ids[i] with n_tokens[i] new tokens (flattened in
  // `tokens`) and n_want[i] wanted places among them (flattened in `want`).  The parts are written one after
  // the other into `out`: token ids, positions, entry of token, cu_q, first position, state slot, wanted rows,
  // tiles of 16 prompt tokens as (entry, offset), rows of single tokens, then per group the cache slot of every
  // token and the block tables [n_entries, width].  table_width < 0: the widest table of the batch (at least 1);
  // else every table is written that wide: a request may hold more pages than that (a prompt's pages are
  // reserved whole while its first portions run), as long as the pages up to its last token of this step fit,
  // since no later one is read or written in the step.
  // padded: null, or five counts (tokens, entries, wanted places, tiles, single rows), each at least what the batch
  // has, up to which the description is filled with parts that do nothing (a token without entry or slot, an entry
  // without rows, a tile in such an entry, a single row of -1, a wanted place that is row 0): steps whose counts
  // differ a little then share one layout.  More tiles than the batch has need at least one entry more.
  // sizes: 9 + 2 * groups part lengths; widths: per group.  Returns the total length or a CacheStatus.
  int64_t pack_batch(int n_entries, const int64_t* ids, const int* n_tokens, const int32_t* tokens,
                     const int* n_want, const int* want, int table_width, const int64_t* padded, int32_t* out,
                     int64_t capacity, int64_t* sizes, int* widths, int* entry_info) const;

 private:
  Request* find(int64_t id);
  int page_size_, max_requests_;
  bool prefix_cache_;
  std::vector<std::unique_ptr<Group>> groups_;
  std::vector<int> free_slots_;
  std::unordered_map<int64_t, Request> requests_;
};

}  // namespace ta
