// Page allocator of the key/value cache: free stack, reference counts, an index of full pages by the hash
// of their tokens, and the pages that index keeps findable after their last holder has gone (oldest first).
// Behaviour follows qwen-infer/src/paged.rs:125-519: page ids are 0..n-1, the first allocation returns 0,
// the page freed last is handed out next, and an allocation evicts cached pages only once the free stack
// is empty.
#pragma once
#include <cstdint>
#include <list>
#include <string>
#include <unordered_map>
#include <vector>

namespace ta {

enum Release { RELEASE_SHARED = 0, RELEASE_CACHED = 1, RELEASE_FREED = 2 };
enum AllocStatus { ALLOC_OK = 0, ALLOC_DOUBLE_FREE = -1, ALLOC_UNKNOWN_PAGE = -2, ALLOC_NOT_FULL = -3 };

// Chained hash of one full page of token ids (qwen-infer/src/paged.rs:93-100).
uint64_t prefix_page_hash(uint64_t parent, const int32_t* tokens, int count);

class PageAllocator {
 public:
  PageAllocator(int num_pages, int page_size);

  int page_size() const { return page_size_; }
  int capacity() const { return capacity_; }
  int free_count() const { return (int)free_.size(); }
  int cached_count() const { return (int)cached_.size(); }
  int available() const { return free_count() + cached_count(); }
  int live_count() const { return live_; }
  int occupied() const { return live_ + cached_count(); }
  int refcount(int page) const { return known(page) ? refcount_[page] : -1; }
  bool all_refcounts_zero() const { return live_ == 0; }
  int peak_live() const { return peak_live_; }
  int peak_occupied() const { return peak_occupied_; }
  void rewind_peaks(int live, int occupied);

  int alloc();                                            // a page id, or -1
  bool alloc_n(int count, std::vector<int>* out);         // `count` pages appended to `out`, or none at all
  int free_page(int page, int* how);                      // AllocStatus; *how = Release
  int incref(int page);                                   // AllocStatus

  int publish_full_page(uint64_t parent_hash, const int32_t* tokens, int count, int page);
  int find_full_page(uint64_t parent_hash, int parent_page, const int32_t* tokens, int count) const;   // or -1
  void take_shared_prefix(const int32_t* tokens, int count, std::vector<int>* out);
  void publish_prompt_pages(const int32_t* tokens, int count, const int* pages, int n_pages);
  void reclaim_cached();
  std::string check_invariants() const;                   // empty when all is well

  // The index under a given hash value (what the calls above do after hashing; tests use them to make two
  // different pages meet under one value).  tokens: one full page.
  bool publish_at(uint64_t value, uint64_t parent_hash, int parent_page, const int32_t* tokens, int page);
  int find_at(uint64_t value, uint64_t parent_hash, int parent_page, const int32_t* tokens) const;

 private:
  struct Entry {
    int page;
    uint64_t parent_hash;
    int parent_page;                                      // -1: none
    std::vector<int32_t> tokens;
  };
  bool known(int page) const { return page >= 0 && page < capacity_; }
  void note_peaks();
  void unindex(int page);
  void uncache(int page);

  int page_size_, capacity_;
  std::vector<int> free_;                                 // a stack: back() is handed out next
  std::vector<int> refcount_;
  std::vector<char> has_hash_;
  std::vector<uint64_t> hash_of_;
  std::list<int> cached_;                                 // oldest first
  std::vector<std::list<int>::iterator> cached_at_;
  std::vector<char> is_cached_;
  std::unordered_map<uint64_t, Entry> index_;
  int live_ = 0, peak_live_ = 0, peak_occupied_ = 0;
};

}  // namespace ta
