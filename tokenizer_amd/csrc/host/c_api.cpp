// C entry points of the host library (bound from Python through ctypes).  Objects are opaque pointers;
// functions return a status or a value as their headers say; `ta_host_message` holds the text of the last
// failed check of the calling thread.
#include <cstring>
#include <string>

#include "bpe_core.h"
#include "cache_core.h"
#include "page_allocator.h"
#include "sampler.h"
#include "scheduler_core.h"

using namespace ta;

static thread_local std::string g_message;

extern "C" {

const char* ta_host_message() { return g_message.c_str(); }

// ---------------------------------------------------------------------------------------- allocator
void* ta_alloc_new(int num_pages, int page_size) {
  if (num_pages < 0 || page_size <= 0) return nullptr;
  return new PageAllocator(num_pages, page_size);
}
void ta_alloc_delete(void* a) { delete (PageAllocator*)a; }
// what: 0 capacity, 1 free, 2 cached, 3 available, 4 live, 5 occupied, 6 refcount(arg), 7 all counts zero,
// 8 peak live, 9 peak occupied, 10 page size.
int ta_alloc_get(void* a, int what, int arg) {
  const PageAllocator& p = *(PageAllocator*)a;
  switch (what) {
    case 0: return p.capacity();
    case 1: return p.free_count();
    case 2: return p.cached_count();
    case 3: return p.available();
    case 4: return p.live_count();
    case 5: return p.occupied();
    case 6: return p.refcount(arg);
    case 7: return p.all_refcounts_zero() ? 1 : 0;
    case 8: return p.peak_live();
    case 9: return p.peak_occupied();
    case 10: return p.page_size();
    default: return -1;
  }
}
void ta_alloc_rewind_peaks(void* a, int live, int occupied) { ((PageAllocator*)a)->rewind_peaks(live, occupied); }
int ta_alloc_alloc(void* a) { return ((PageAllocator*)a)->alloc(); }
// `count` pages into out, or none: returns 1 or 0.
int ta_alloc_alloc_n(void* a, int count, int* out) {
  std::vector<int> pages;
  if (!((PageAllocator*)a)->alloc_n(count, &pages)) return 0;
  std::copy(pages.begin(), pages.end(), out);
  return 1;
}
int ta_alloc_free(void* a, int page, int* how) { return ((PageAllocator*)a)->free_page(page, how); }
int ta_alloc_incref(void* a, int page) { return ((PageAllocator*)a)->incref(page); }
uint64_t ta_prefix_page_hash(uint64_t parent, const int32_t* tokens, int count) {
  return prefix_page_hash(parent, tokens, count);
}
int ta_alloc_publish_full_page(void* a, uint64_t parent_hash, const int32_t* tokens, int count, int page) {
  return ((PageAllocator*)a)->publish_full_page(parent_hash, tokens, count, page);
}
int ta_alloc_find_full_page(void* a, uint64_t parent_hash, int parent_page, const int32_t* tokens, int count) {
  return ((PageAllocator*)a)->find_full_page(parent_hash, parent_page, tokens, count);
}
int ta_alloc_publish_at(void* a, uint64_t value, uint64_t parent_hash, int parent_page, const int32_t* tokens,
                        int count, int page) {
  PageAllocator& p = *(PageAllocator*)a;
  if (count != p.page_size() || p.refcount(page) < 0) return 0;
  return p.publish_at(value, parent_hash, parent_page, tokens, page) ? 1 : 0;
}
int ta_alloc_find_at(void* a, uint64_t value, uint64_t parent_hash, int parent_page, const int32_t* tokens, int count) {
  const PageAllocator& p = *(PageAllocator*)a;
  return count == p.page_size() ? p.find_at(value, parent_hash, parent_page, tokens) : -1;
}
// Pages into out (room for count / page_size); returns how many.
int ta_alloc_take_shared_prefix(void* a, const int32_t* tokens, int count, int* out) {
  std::vector<int> pages;
  ((PageAllocator*)a)->take_shared_prefix(tokens, count, &pages);
  std::copy(pages.begin(), pages.end(), out);
  return (int)pages.size();
}
void ta_alloc_publish_prompt_pages(void* a, const int32_t* tokens, int count, const int* pages, int n_pages) {
  ((PageAllocator*)a)->publish_prompt_pages(tokens, count, pages, n_pages);
}
void ta_alloc_reclaim_cached(void* a) { ((PageAllocator*)a)->reclaim_cached(); }
// 0 when all is well, else 1 with the finding in ta_host_message().
int ta_alloc_check(void* a) {
  g_message = ((PageAllocator*)a)->check_invariants();
  return g_message.empty() ? 0 : 1;
}

// ------------------------------------------------------------------------------------------- cache
// windows[g] < 0: group g keeps every position; else the window behind which its pages are given back.
void* ta_cache_new(int n_groups, const int* windows, int num_pages, int page_size, int max_requests,
                   int prefix_cache, int n_state_layers) {
  if (n_groups < 0 || num_pages < 0 || page_size <= 0 || max_requests < 0 || n_state_layers < 0) return nullptr;
  return new CacheCore(n_groups, windows, num_pages, page_size, max_requests, prefix_cache != 0, n_state_layers);
}
void ta_cache_delete(void* c) { delete (CacheCore*)c; }
void* ta_cache_allocator(void* c, int group) { return ((CacheCore*)c)->allocator(group); }   // borrowed
int ta_cache_prefix_enabled(void* c) { return ((CacheCore*)c)->prefix_cache() ? 1 : 0; }
int ta_cache_n_requests(void* c) { return ((CacheCore*)c)->n_requests(); }
int ta_cache_free_slots(void* c) { return ((CacheCore*)c)->free_slot_count(); }
// The ids of the live requests into out (room for ta_cache_n_requests); returns how many.
int ta_cache_request_ids(void* c, int64_t* out) { return ((CacheCore*)c)->request_ids(out); }
int ta_cache_add_request(void* c, int64_t id) { return ((CacheCore*)c)->add_request(id); }
int ta_cache_has_request(void* c, int64_t id) { return ((const CacheCore*)c)->find(id) ? 1 : 0; }
int ta_cache_seq_len(void* c, int64_t id) {
  const Request* r = ((const CacheCore*)c)->find(id);
  return r ? r->seq_len : CACHE_UNKNOWN_REQUEST;
}
int ta_cache_slot(void* c, int64_t id) {
  const Request* r = ((const CacheCore*)c)->find(id);
  return r ? r->slot : CACHE_UNKNOWN_REQUEST;
}
int ta_cache_table_len(void* c, int64_t id, int group) {
  const Request* r = ((const CacheCore*)c)->find(id);
  return r ? (int)r->tables[group].size() : CACHE_UNKNOWN_REQUEST;
}
int ta_cache_table(void* c, int64_t id, int group, int* out) {
  const Request* r = ((const CacheCore*)c)->find(id);
  if (!r) return CACHE_UNKNOWN_REQUEST;
  std::copy(r->tables[group].begin(), r->tables[group].end(), out);
  return (int)r->tables[group].size();
}
int ta_cache_first_needed_position(void* c, int group, int seq_len) {
  return ((CacheCore*)c)->first_needed_position(group, seq_len);
}
int ta_cache_pages_missing(void* c, int64_t id, int new_len, int* per_group) {
  return ((CacheCore*)c)->pages_missing(id, new_len, per_group);
}
int ta_cache_can_reserve(void* c, int64_t id, int new_len) { return ((CacheCore*)c)->can_reserve(id, new_len); }
int ta_cache_reserve(void* c, int64_t id, int new_len) { return ((CacheCore*)c)->reserve(id, new_len); }
int ta_cache_advance(void* c, int64_t id, int new_len) { return ((CacheCore*)c)->advance(id, new_len); }
int ta_cache_release(void* c, int64_t id) { return ((CacheCore*)c)->release(id); }
int ta_cache_detach(void* c, int64_t id) { return ((CacheCore*)c)->detach(id); }
int ta_cache_attach_shared_prefix(void* c, int64_t id, const int32_t* tokens, int count) {
  return ((CacheCore*)c)->attach_shared_prefix(id, tokens, count);
}
int ta_cache_publish(void* c, int64_t id, const int32_t* tokens, int count) {
  return ((CacheCore*)c)->publish(id, tokens, count);
}
int ta_cache_check(void* c) {
  g_message = ((CacheCore*)c)->check_invariants();
  return g_message.empty() ? 0 : 1;
}
int64_t ta_cache_pack_batch(void* c, int n_entries, const int64_t* ids, const int* n_tokens, const int32_t* tokens,
                            const int* n_want, const int* want, int table_width, const int64_t* padded, int32_t* out,
                            int64_t capacity, int64_t* sizes, int* widths, int* entry_info) {
  return ((CacheCore*)c)->pack_batch(n_entries, ids, n_tokens, tokens, n_want, want, table_width, padded, out, capacity,
                                     sizes, widths, entry_info);
}

// ---------------------------------------------------------------------------------------- scheduler
void* ta_sched_new(void* cache, int num_pages, int max_batch_size, int token_budget, int prefill_chunk,
                   int prompts_first) {
  if (!cache || max_batch_size <= 0 || token_budget <= 0) return nullptr;
  return new SchedulerCore((CacheCore*)cache, num_pages, max_batch_size, token_budget, prefill_chunk,
                           prompts_first != 0);
}
void ta_sched_delete(void* s) { delete (SchedulerCore*)s; }
int ta_sched_enqueue(void* s, int64_t id, const int32_t* prompt, int count) {
  return ((SchedulerCore*)s)->enqueue(id, prompt, count);
}
int ta_sched_append_token(void* s, int64_t id, int32_t token) { return ((SchedulerCore*)s)->append_token(id, token); }
// what: 0 running, 1 waiting, 2 most running at once, 3 preemptions, 4 last preempted id, 5 front of the queue
// (-1: empty), 6 pages to admit `id`, 7 tokens of `id` in the cache, 8 tokens `id` holds, 9 whether `id` runs.
int64_t ta_sched_get(void* s, int what, int64_t id) {
  const SchedulerCore& core = *(SchedulerCore*)s;
  const Sequence* seq = what >= 7 && what <= 9 ? core.find(id) : nullptr;
  switch (what) {
    case 0: return core.n_running();
    case 1: return core.n_waiting();
    case 2: return core.max_running();
    case 3: return core.preemptions();
    case 4: return core.last_preempted_id();
    case 5: return core.front_waiting();
    case 6: return core.pages_to_admit(id);
    case 7: return seq ? seq->computed : -1;
    case 8: return seq ? (int64_t)seq->tokens.size() : -1;
    case 9: return seq ? (seq->running ? 1 : 0) : -1;
    case 10: return core.prefix_hits();
    case 11: return core.prefix_tokens_reused();
    default: return -1;
  }
}
// planned: rows of (id, first token, count, completes); preempted: ids; failed: rows of (id, pages needed).
// Each array has room for `room` rows.  Returns 0, or -1 if a list did not fit (nothing is lost: the lists are
// never longer than the number of sequences the scheduler knows, which the caller passes as `room`).
int ta_sched_plan_step(void* s, int room, int64_t* planned, int* n_planned, int64_t* preempted, int* n_preempted,
                       int64_t* failed, int* n_failed) {
  std::vector<PlannedEntry> plan;
  std::vector<int64_t> out;
  std::vector<FailedEntry> fail;
  ((SchedulerCore*)s)->plan_step(&plan, &out, &fail);
  *n_planned = (int)plan.size(); *n_preempted = (int)out.size(); *n_failed = (int)fail.size();
  if ((int)plan.size() > room || (int)out.size() > room || (int)fail.size() > room) return -1;
  for (size_t i = 0; i < plan.size(); ++i) {
    planned[4 * i] = plan[i].id; planned[4 * i + 1] = plan[i].first; planned[4 * i + 2] = plan[i].count;
    planned[4 * i + 3] = plan[i].completes ? 1 : 0;
  }
  std::copy(out.begin(), out.end(), preempted);
  for (size_t i = 0; i < fail.size(); ++i) { failed[2 * i] = fail[i].id; failed[2 * i + 1] = fail[i].pages_needed; }
  return 0;
}
// The running (which = 0, in order of admission) or waiting (1, front first) ids into out; returns how many.
int ta_sched_list(void* s, int which, int64_t* out) {
  const SchedulerCore& core = *(SchedulerCore*)s;
  if (which == 0) { std::copy(core.running().begin(), core.running().end(), out); return (int)core.running().size(); }
  std::copy(core.waiting().begin(), core.waiting().end(), out);
  return (int)core.waiting().size();
}
int ta_sched_tokens(void* s, int64_t id, int first, int count, int32_t* out) {
  const Sequence* seq = ((const SchedulerCore*)s)->find(id);
  if (!seq || first < 0 || count < 0 || first + count > (int)seq->tokens.size()) return -1;
  std::copy(seq->tokens.begin() + first, seq->tokens.begin() + first + count, out);
  return count;
}
int ta_sched_commit(void* s, int64_t id, int count) { return ((SchedulerCore*)s)->commit(id, count); }
int ta_sched_finish(void* s, int64_t id) { return ((SchedulerCore*)s)->finish(id); }

// ----------------------------------------------------------------------------------------- sampling
float ta_uniform_f32(uint64_t seed, uint64_t counter) { return uniform_f32(seed, counter); }
int ta_greedy_token(const float* logits, int64_t count) { return greedy_token(logits, count); }
int ta_sample_with_uniform(const float* logits, int64_t count, float temperature, float top_p, float uniform) {
  return sample_with_uniform(logits, count, temperature, top_p, uniform);
}

// ---------------------------------------------------------------------------------------- tokenizer
void* ta_bpe_new() { return new BpeCore(); }
void ta_bpe_delete(void* b) { delete (BpeCore*)b; }
int ta_bpe_add_token(void* b, int32_t id, const uint8_t* bytes, int len, int findable) {
  return ((BpeCore*)b)->add_token(id, bytes, len, findable != 0);
}
int ta_bpe_add_merge(void* b, const uint8_t* merged, int len, int rank) {
  return ((BpeCore*)b)->add_merge(merged, len, rank);
}
int ta_bpe_vocab_size(void* b) { return ((BpeCore*)b)->vocab_size(); }
int ta_bpe_encode_piece(void* b, const uint8_t* piece, int len, int32_t* out, int capacity) {
  return ((BpeCore*)b)->encode_piece(piece, len, out, capacity);
}
int64_t ta_bpe_decode(void* b, const int32_t* ids, int count, uint8_t* out, int64_t capacity, int* bad_at) {
  return ((BpeCore*)b)->decode(ids, count, out, capacity, bad_at);
}

}  // extern "C"
