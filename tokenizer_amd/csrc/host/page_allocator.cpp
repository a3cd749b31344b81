#include "page_allocator.h"

#include <algorithm>
#include <cstring>

namespace ta {

uint64_t prefix_page_hash(uint64_t parent, const int32_t* tokens, int count) {
  uint64_t value = 0xCBF29CE484222325ull ^ parent;
  for (int i = 0; i < count; ++i) {
    value ^= (uint64_t)(uint32_t)tokens[i];
    value *= 0x100000001B3ull;
  }
  return value;
}

PageAllocator::PageAllocator(int num_pages, int page_size)
    : page_size_(page_size), capacity_(num_pages), refcount_(num_pages, 0), has_hash_(num_pages, 0),
      hash_of_(num_pages, 0), cached_at_(num_pages), is_cached_(num_pages, 0) {
  free_.reserve(num_pages);
  for (int page = num_pages - 1; page >= 0; --page) free_.push_back(page);
}

void PageAllocator::note_peaks() {
  peak_live_ = std::max(peak_live_, live_);
  peak_occupied_ = std::max(peak_occupied_, occupied());
}

void PageAllocator::rewind_peaks(int live, int occ) {
  peak_live_ = std::max(live, live_);
  peak_occupied_ = std::max(occ, occupied());
}

void PageAllocator::uncache(int page) {
  cached_.erase(cached_at_[page]);
  is_cached_[page] = 0;
}

int PageAllocator::alloc() {
  int page;
  if (!free_.empty()) {
    page = free_.back();
    free_.pop_back();
  } else if (!cached_.empty()) {
    page = cached_.front();
    uncache(page);
    unindex(page);
  } else {
    return -1;
  }
  refcount_[page] = 1;
  ++live_;
  note_peaks();
  return page;
}

bool PageAllocator::alloc_n(int count, std::vector<int>* out) {
  if (available() < count) return false;
  for (int i = 0; i < count; ++i) out->push_back(alloc());
  return true;
}

int PageAllocator::free_page(int page, int* how) {
  if (!known(page)) return ALLOC_UNKNOWN_PAGE;
  if (refcount_[page] == 0) return ALLOC_DOUBLE_FREE;
  if (--refcount_[page] > 0) {
    if (how) *how = RELEASE_SHARED;
    return ALLOC_OK;
  }
  --live_;
  if (has_hash_[page]) {
    cached_.push_back(page);
    cached_at_[page] = std::prev(cached_.end());
    is_cached_[page] = 1;
    if (how) *how = RELEASE_CACHED;
  } else {
    free_.push_back(page);
    if (how) *how = RELEASE_FREED;
  }
  note_peaks();
  return ALLOC_OK;
}

int PageAllocator::incref(int page) {
  if (!known(page)) return ALLOC_UNKNOWN_PAGE;
  if (refcount_[page] == 0) {
    if (!is_cached_[page]) return ALLOC_DOUBLE_FREE;
    uncache(page);
    refcount_[page] = 1;
    ++live_;
    note_peaks();
    return ALLOC_OK;
  }
  ++refcount_[page];
  return ALLOC_OK;
}

bool PageAllocator::publish_at(uint64_t value, uint64_t parent_hash, int parent_page, const int32_t* tokens,
                               int page) {
  auto found = index_.find(value);
  if (found != index_.end()) {
    const Entry& e = found->second;
    return e.page == page && e.parent_hash == parent_hash && e.parent_page == parent_page &&
           std::equal(e.tokens.begin(), e.tokens.end(), tokens);
  }
  if (has_hash_[page]) return false;
  index_.emplace(value, Entry{page, parent_hash, parent_page, std::vector<int32_t>(tokens, tokens + page_size_)});
  has_hash_[page] = 1;
  hash_of_[page] = value;
  return true;
}

int PageAllocator::find_at(uint64_t value, uint64_t parent_hash, int parent_page, const int32_t* tokens) const {
  auto found = index_.find(value);
  if (found == index_.end()) return -1;
  const Entry& e = found->second;
  if (e.parent_hash != parent_hash || e.parent_page != parent_page ||
      !std::equal(e.tokens.begin(), e.tokens.end(), tokens))
    return -1;
  return e.page;
}

void PageAllocator::unindex(int page) {
  if (!has_hash_[page]) return;
  has_hash_[page] = 0;
  auto found = index_.find(hash_of_[page]);
  if (found != index_.end() && found->second.page == page) index_.erase(found);
}

int PageAllocator::publish_full_page(uint64_t parent_hash, const int32_t* tokens, int count, int page) {
  if (count != page_size_) return ALLOC_NOT_FULL;
  if (!known(page) || refcount_[page] == 0) return ALLOC_UNKNOWN_PAGE;
  publish_at(prefix_page_hash(parent_hash, tokens, count), parent_hash, -1, tokens, page);
  return ALLOC_OK;
}

int PageAllocator::find_full_page(uint64_t parent_hash, int parent_page, const int32_t* tokens, int count) const {
  if (count != page_size_) return -1;
  return find_at(prefix_page_hash(parent_hash, tokens, count), parent_hash, parent_page, tokens);
}

void PageAllocator::take_shared_prefix(const int32_t* tokens, int count, std::vector<int>* out) {
  uint64_t parent_hash = 0;
  int parent_page = -1;
  for (int offset = 0; offset + page_size_ <= count; offset += page_size_) {
    const int32_t* chunk = tokens + offset;
    const int page = find_full_page(parent_hash, parent_page, chunk, page_size_);
    if (page < 0 || incref(page) != ALLOC_OK) break;
    out->push_back(page);
    parent_hash = prefix_page_hash(parent_hash, chunk, page_size_);
    parent_page = page;
  }
}

void PageAllocator::publish_prompt_pages(const int32_t* tokens, int count, const int* pages, int n_pages) {
  uint64_t parent_hash = 0;
  int parent_page = -1;
  for (int index = 0; index < count / page_size_ && index < n_pages; ++index) {
    const int32_t* chunk = tokens + (size_t)index * page_size_;
    const int page = pages[index];
    const uint64_t value = prefix_page_hash(parent_hash, chunk, page_size_);
    if (!known(page) || refcount_[page] == 0) break;
    publish_at(value, parent_hash, parent_page, chunk, page);
    if (find_at(value, parent_hash, parent_page, chunk) != page) break;
    parent_hash = value;
    parent_page = page;
  }
}

void PageAllocator::reclaim_cached() {
  while (!cached_.empty()) {
    const int page = cached_.front();
    uncache(page);
    unindex(page);
    free_.push_back(page);
  }
}

std::string PageAllocator::check_invariants() const {
  std::vector<int> on_stack(capacity_, 0);
  for (int page : free_) {
    if (!known(page)) return "a page outside the pool is on the free stack";
    if (++on_stack[page] > 1) return "a page is on the free stack twice";
  }
  int live = 0;
  for (int page = 0; page < capacity_; ++page) {
    const int places = on_stack[page] + (is_cached_[page] ? 1 : 0) + (refcount_[page] > 0 ? 1 : 0);
    if (places != 1) return "page " + std::to_string(page) + " is in " + std::to_string(places) + " places";
    if (is_cached_[page] && !has_hash_[page]) return "a cached page has no hash";
    live += refcount_[page] > 0;
  }
  if (live != live_) return "the count of live pages is off";
  return "";
}

}  // namespace ta
