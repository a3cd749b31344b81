#include "cache_core.h"

#include <algorithm>

namespace ta {

static int pages_for_len(int length, int page_size) { return (length + page_size - 1) / page_size; }

CacheCore::CacheCore(int n_groups, const int* windows, int num_pages, int page_size, int max_requests,
                     bool prefix_cache, int n_state_layers)
    : page_size_(page_size), max_requests_(max_requests) {
  bool all_kept = true;
  for (int g = 0; g < n_groups; ++g) {
    groups_.emplace_back(new Group(windows[g], num_pages, page_size));
    all_kept = all_kept && groups_.back()->keeps_all();
  }
  // Sharing a prefix needs every group to keep all positions (a window group drops pages) and no layer with
  // state of its own in the slot (it would never see the tokens of an attached prefix).
  prefix_cache_ = prefix_cache && all_kept && n_state_layers == 0;
  for (int slot = max_requests - 1; slot >= 0; --slot) free_slots_.push_back(slot);
}

const Request* CacheCore::find(int64_t id) const {
  auto found = requests_.find(id);
  return found == requests_.end() ? nullptr : &found->second;
}

int CacheCore::request_ids(int64_t* out) const {
  int count = 0;
  for (const auto& item : requests_) out[count++] = item.first;
  std::sort(out, out + count);
  return count;
}

Request* CacheCore::find(int64_t id) {
  auto found = requests_.find(id);
  return found == requests_.end() ? nullptr : &found->second;
}

int CacheCore::add_request(int64_t id) {
  if (requests_.count(id)) return CACHE_ALREADY_LIVE;
  if (free_slots_.empty()) return CACHE_NO_SLOT;
  Request request;
  request.slot = free_slots_.back();
  free_slots_.pop_back();
  request.tables.resize(groups_.size());
  const int slot = request.slot;
  requests_.emplace(id, std::move(request));
  return slot;
}

int CacheCore::first_needed_position(int group, int seq_len) const {
  const Group& g = *groups_[group];
  return g.keeps_all() ? 0 : std::max(0, seq_len - g.window);
}

int CacheCore::pages_missing(int64_t id, int new_len, int* per_group) const {
  const Request* request = find(id);
  if (!request) return CACHE_UNKNOWN_REQUEST;
  for (size_t g = 0; g < groups_.size(); ++g)
    per_group[g] = std::max(0, pages_for_len(new_len, page_size_) - (int)request->tables[g].size());
  return CACHE_OK;
}

int CacheCore::can_reserve(int64_t id, int new_len) const {
  std::vector<int> missing(groups_.size());
  const int status = pages_missing(id, new_len, missing.data());
  if (status != CACHE_OK) return status;
  for (size_t g = 0; g < groups_.size(); ++g)
    if (groups_[g]->allocator.available() < missing[g]) return 0;
  return 1;
}

int CacheCore::reserve(int64_t id, int new_len) {
  const int possible = can_reserve(id, new_len);
  if (possible != 1) return possible;
  Request* request = find(id);
  for (size_t g = 0; g < groups_.size(); ++g) {
    const int missing = std::max(0, pages_for_len(new_len, page_size_) - (int)request->tables[g].size());
    groups_[g]->allocator.alloc_n(missing, &request->tables[g]);
  }
  return 1;
}

int CacheCore::advance(int64_t id, int new_len) {
  Request* request = find(id);
  if (!request) return CACHE_UNKNOWN_REQUEST;
  if (new_len < request->seq_len) return CACHE_SHRINKS;
  for (const auto& table : request->tables)
    if (pages_for_len(new_len, page_size_) > (int)table.size()) return CACHE_TOO_FEW_PAGES;
  request->seq_len = new_len;
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g]->keeps_all()) continue;
    // Pages no later query reads again go back to the pool.
    const int first = first_needed_position((int)g, new_len);
    std::vector<int>& table = request->tables[g];
    for (int index = 0; index < first / page_size_; ++index) {
      if (table[index] >= 0) {
        groups_[g]->allocator.free_page(table[index], nullptr);
        table[index] = -1;
      }
    }
  }
  return CACHE_OK;
}

static void free_table(Group& group, std::vector<int>& table) {
  for (int page : table)
    if (page >= 0) group.allocator.free_page(page, nullptr);
}

int CacheCore::release(int64_t id) {
  auto found = requests_.find(id);
  if (found == requests_.end()) return CACHE_UNKNOWN_REQUEST;
  for (size_t g = 0; g < groups_.size(); ++g) free_table(*groups_[g], found->second.tables[g]);
  free_slots_.push_back(found->second.slot);
  requests_.erase(found);
  return CACHE_OK;
}

int CacheCore::detach(int64_t id) {
  Request* request = find(id);
  if (!request) return CACHE_UNKNOWN_REQUEST;
  for (size_t g = 0; g < groups_.size(); ++g) {
    free_table(*groups_[g], request->tables[g]);
    request->tables[g].clear();
  }
  request->seq_len = 0;
  return CACHE_OK;
}

int CacheCore::attach_shared_prefix(int64_t id, const int32_t* tokens, int count) {
  Request* request = find(id);
  if (!request) return CACHE_UNKNOWN_REQUEST;
  if (!prefix_cache_ || request->seq_len) return 0;
  for (const auto& table : request->tables)
    if (!table.empty()) return 0;
  // The last token is left out of the lookup so that the page it lands in stays private
  // (qwen-server/src/engine.rs:490-495,519-527).
  const int lookup = count > 0 ? count - 1 : 0;
  std::vector<std::vector<int>> taken(groups_.size());
  std::vector<std::pair<int, int>> marks;
  for (size_t g = 0; g < groups_.size(); ++g) {
    PageAllocator& allocator = groups_[g]->allocator;
    marks.emplace_back(allocator.peak_live(), allocator.peak_occupied());
    allocator.take_shared_prefix(tokens, lookup, &taken[g]);
  }
  size_t shared = taken.empty() ? 0 : taken[0].size();
  for (const auto& pages : taken) shared = std::min(shared, pages.size());
  for (size_t g = 0; g < groups_.size(); ++g) {
    PageAllocator& allocator = groups_[g]->allocator;
    for (size_t i = shared; i < taken[g].size(); ++i) allocator.free_page(taken[g][i], nullptr);
    if (taken[g].size() > shared) allocator.rewind_peaks(marks[g].first, marks[g].second);
    request->tables[g].insert(request->tables[g].end(), taken[g].begin(), taken[g].begin() + shared);
  }
  request->seq_len = (int)shared * page_size_;
  return request->seq_len;
}

int CacheCore::publish(int64_t id, const int32_t* tokens, int count) {
  if (!prefix_cache_) return CACHE_OK;
  const Request* request = find(id);
  if (!request) return CACHE_UNKNOWN_REQUEST;
  const int written = std::min(count, request->seq_len);
  for (size_t g = 0; g < groups_.size(); ++g)
    groups_[g]->allocator.publish_prompt_pages(tokens, written, request->tables[g].data(),
                                               (int)request->tables[g].size());
  return CACHE_OK;
}

std::string CacheCore::check_invariants() const {
  for (size_t g = 0; g < groups_.size(); ++g) {
    const PageAllocator& allocator = groups_[g]->allocator;
    std::string fault = allocator.check_invariants();
    if (!fault.empty()) return "group " + std::to_string(g) + ": " + fault;
    std::vector<int> held(allocator.capacity(), 0);
    for (const auto& item : requests_)
      for (int page : item.second.tables[g])
        if (page >= 0) ++held[page];
    for (int page = 0; page < allocator.capacity(); ++page)
      if (allocator.refcount(page) != held[page])
        return "group " + std::to_string(g) + " page " + std::to_string(page) + ": count " +
               std::to_string(allocator.refcount(page)) + ", held " + std::to_string(held[page]);
    if (allocator.free_count() + allocator.cached_count() + allocator.live_count() != allocator.capacity())
      return "group " + std::to_string(g) + ": pages do not add up";
  }
  std::vector<int> slots(max_requests_, 0);
  for (const auto& item : requests_) {
    const int slot = item.second.slot;
    if (slot < 0 || slot >= max_requests_ || ++slots[slot] > 1) return "a slot is held twice";
  }
  for (int slot : free_slots_)
    if (slot < 0 || slot >= max_requests_ || ++slots[slot] > 1) return "a slot is free and held, or free twice";
  for (int count : slots)
    if (count != 1) return "a slot was lost";
  return "";
}

int64_t CacheCore::pack_batch(int n_entries, const int64_t* ids, const int* n_tokens, const int32_t* tokens,
                              const int* n_want, const int* want, int table_width, const int64_t* padded,
                              int32_t* out, int64_t capacity, int64_t* sizes, int* widths, int* entry_info) const {
  const int n_groups = (int)groups_.size();
  std::vector<const Request*> requests(n_entries);
  int64_t real_tokens = 0, real_want = 0, real_tiles = 0, real_single = 0;
  for (int e = 0; e < n_entries; ++e) {
    requests[e] = find(ids[e]);
    if (!requests[e]) return CACHE_UNKNOWN_REQUEST;
    if (n_tokens[e] <= 0 || n_want[e] < 0) return CACHE_BAD_ARGUMENT;
    real_tokens += n_tokens[e];
    real_want += n_want[e];
    if (n_tokens[e] == 1) ++real_single; else real_tiles += (n_tokens[e] + 15) / 16;
  }
  // The description may be filled up to given counts (tokens, entries, wanted places, tiles, single rows) with
  // parts that do nothing: so that steps whose counts differ a little have the same layout and launch sizes.
  // A token past the real ones has id 0, position 0, no entry (-1) and no slot (-1); an entry past the real ones
  // has no rows and a table of -1; a wanted place past the real ones is row 0; a tile past the real ones lies in
  // the first such entry (no rows: kernels pass it over) and a single row past the real ones is -1.
  const int n_real_entries = n_entries;
  int64_t total_tokens = real_tokens, total_want = real_want, n_tiles = real_tiles, n_single = real_single;
  if (padded) {
    if (padded[0] < real_tokens || padded[1] < n_entries || padded[2] < real_want || padded[3] < real_tiles ||
        padded[4] < real_single || (padded[3] > real_tiles && padded[1] == n_entries))
      return CACHE_BAD_ARGUMENT;
    total_tokens = padded[0]; n_entries = (int)padded[1]; total_want = padded[2]; n_tiles = padded[3]; n_single = padded[4];
  }
  for (int g = 0; g < n_groups; ++g) {
    int width = 1;
    if (table_width >= 0) {
      // A fixed width has to hold the pages up to each request's last token of this step; pages a request holds
      // beyond that are left out.
      for (int e = 0; e < n_real_entries; ++e)
        if (pages_for_len(requests[e]->seq_len + n_tokens[e], page_size_) > table_width) return CACHE_TABLE_TOO_WIDE;
      width = table_width;
    } else {
      for (int e = 0; e < n_real_entries; ++e) width = std::max(width, (int)requests[e]->tables[g].size());
    }
    widths[g] = width;
  }
  int64_t* size = sizes;
  *size++ = total_tokens; *size++ = total_tokens; *size++ = total_tokens; *size++ = n_entries + 1;
  *size++ = n_entries; *size++ = n_entries; *size++ = total_want; *size++ = 2 * n_tiles; *size++ = n_single;
  for (int g = 0; g < n_groups; ++g) { *size++ = total_tokens; *size++ = (int64_t)n_entries * widths[g]; }
  int64_t total = 0;
  for (int i = 0; i < 9 + 2 * n_groups; ++i) total += sizes[i];
  if (total > capacity) return CACHE_BUFFER_TOO_SMALL;

  int32_t* token_ids = out;
  int32_t* positions = token_ids + total_tokens;
  int32_t* entry_of_token = positions + total_tokens;
  int32_t* cu_q = entry_of_token + total_tokens;
  int32_t* first_position = cu_q + n_entries + 1;
  int32_t* state_slots = first_position + n_entries;
  int32_t* want_rows = state_slots + n_entries;
  int32_t* tiles = want_rows + total_want;
  int32_t* single_rows = tiles + 2 * n_tiles;
  int32_t* group_base = single_rows + n_single;

  int64_t row = 0, token_at = 0, want_at = 0;
  cu_q[0] = 0;
  int32_t* const want_end = want_rows + total_want;
  int32_t* const tiles_end = tiles + 2 * n_tiles;
  int32_t* const single_end = single_rows + n_single;
  for (int e = 0; e < n_real_entries; ++e) {
    const Request& request = *requests[e];
    const int start = request.seq_len, count = n_tokens[e];
    for (int i = 0; i < count; ++i) {
      token_ids[row + i] = tokens[token_at + i];
      positions[row + i] = start + i;
      entry_of_token[row + i] = e;
    }
    for (int i = 0; i < n_want[e]; ++i) *want_rows++ = (int32_t)(row + want[want_at + i]);
    cu_q[e + 1] = (int32_t)(row + count);
    first_position[e] = start;
    state_slots[e] = request.slot;
    if (count == 1) {
      *single_rows++ = (int32_t)row;
    } else {
      for (int offset = 0; offset < count; offset += 16) { *tiles++ = e; *tiles++ = offset; }
    }
    if (entry_info) {
      entry_info[4 * e] = (int)row; entry_info[4 * e + 1] = count; entry_info[4 * e + 2] = start;
      entry_info[4 * e + 3] = request.slot;
    }
    row += count;
    token_at += count;
    want_at += n_want[e];
  }
  for (int64_t t = real_tokens; t < total_tokens; ++t) { token_ids[t] = 0; positions[t] = 0; entry_of_token[t] = -1; }
  for (int e = n_real_entries; e < n_entries; ++e) { cu_q[e + 1] = (int32_t)real_tokens; first_position[e] = 0; state_slots[e] = 0; }
  while (want_rows < want_end) *want_rows++ = 0;
  while (tiles < tiles_end) { *tiles++ = n_real_entries; *tiles++ = 0; }
  while (single_rows < single_end) *single_rows++ = -1;
  for (int g = 0; g < n_groups; ++g) {
    int32_t* slots = group_base;
    int32_t* table_out = slots + total_tokens;
    group_base = table_out + (int64_t)n_entries * widths[g];
    int64_t at = 0;
    std::fill(slots + real_tokens, slots + total_tokens, -1);
    std::fill(table_out + (int64_t)n_real_entries * widths[g], table_out + (int64_t)n_entries * widths[g], -1);
    for (int e = 0; e < n_real_entries; ++e) {
      const std::vector<int>& table = requests[e]->tables[g];
      const int start = requests[e]->seq_len;
      for (int i = 0; i < n_tokens[e]; ++i) {
        const int p = start + i;
        if (p / page_size_ >= (int)table.size()) return CACHE_TOO_FEW_PAGES;
        const int page = table[p / page_size_];
        if (page < 0) return CACHE_PAGE_GIVEN_BACK;
        slots[at++] = page * page_size_ + p % page_size_;
      }
      int32_t* dst = table_out + (int64_t)e * widths[g];
      const size_t copied = std::min(table.size(), (size_t)widths[g]);
      std::copy(table.begin(), table.begin() + copied, dst);
      std::fill(dst + copied, dst + widths[g], -1);
    }
  }
  return total;
}

}  // namespace ta
