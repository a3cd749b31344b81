#include "scheduler_core.h"

#include <algorithm>

namespace ta {

static int pages_for(int length, int page_size) { return (length + page_size - 1) / page_size; }

SchedulerCore::SchedulerCore(CacheCore* cache, int num_pages, int max_batch_size, int token_budget, int prefill_chunk,
                             bool prompts_first)
    : cache_(cache), num_pages_(num_pages), max_batch_size_(max_batch_size), token_budget_(token_budget),
      prefill_chunk_(prefill_chunk > 0 ? prefill_chunk : token_budget), prompts_first_(prompts_first) {}

const Sequence* SchedulerCore::find(int64_t id) const {
  auto found = sequences_.find(id);
  return found == sequences_.end() ? nullptr : &found->second;
}

Sequence* SchedulerCore::find(int64_t id) {
  auto found = sequences_.find(id);
  return found == sequences_.end() ? nullptr : &found->second;
}

int SchedulerCore::enqueue(int64_t id, const int32_t* prompt, int count) {
  if (sequences_.count(id) || count <= 0) return -1;
  Sequence seq;
  seq.id = id;
  seq.prompt_len = count;
  seq.tokens.assign(prompt, prompt + count);
  sequences_.emplace(id, std::move(seq));
  waiting_.push_back(id);
  return 0;
}

int SchedulerCore::append_token(int64_t id, int32_t token) {
  Sequence* seq = find(id);
  if (!seq) return -1;
  seq->tokens.push_back(token);
  return 0;
}

int SchedulerCore::pages_to_admit(int64_t id) const {
  const Sequence* seq = find(id);
  if (!seq) return -1;
  // A new request needs its prompt; one that already sampled also gets room for the next token, so that it is
  // not evicted again at once (engine.rs:696-704).
  return pages_for((int)seq->tokens.size() + (seq->sampled() ? 1 : 0), cache_->page_size());
}

void SchedulerCore::drop_running(int64_t id) {
  running_.erase(std::remove(running_.begin(), running_.end(), id), running_.end());
}

void SchedulerCore::admit(std::vector<FailedEntry>* failed) {
  while (!waiting_.empty() && (int)running_.size() < max_batch_size_) {
    const int64_t id = waiting_.front();
    Sequence& seq = *find(id);
    const int needed = pages_to_admit(id);
    if (needed > num_pages_) {
      waiting_.pop_front();
      failed->push_back({id, needed});
      sequences_.erase(id);
      continue;
    }
    if (cache_->free_slot_count() == 0) break;
    cache_->add_request(id);
    const int shared = cache_->attach_shared_prefix(id, seq.tokens.data(), (int)seq.tokens.size());
    if (cache_->reserve(id, needed * cache_->page_size()) != 1) {
      cache_->release(id);                // gives back the shared pages and the slot
      break;
    }
    waiting_.pop_front();
    if (shared > 0) { ++prefix_hits_; prefix_tokens_ += shared; }
    seq.computed = shared;
    seq.running = true;
    running_.push_back(id);
  }
  max_running_ = std::max(max_running_, (int)running_.size());
}

void SchedulerCore::plan_step(std::vector<PlannedEntry>* planned, std::vector<int64_t>* preempted,
                              std::vector<FailedEntry>* failed) {
  admit(failed);
  if (running_.empty()) return;
  // Oldest first; decoding sequences before prompt portions, or after them.
  std::vector<int64_t> order = running_;
  std::stable_sort(order.begin(), order.end(), [&](int64_t a, int64_t b) {
    const bool da = find(a)->decoding(), db = find(b)->decoding();
    if (da != db) return prompts_first_ ? db : da;
    return a < b;
  });
  int budget = token_budget_;
  for (int64_t id : order) {
    Sequence* seq = find(id);
    if (!seq || !seq->running || budget <= 0) continue;
    const int count = seq->decoding() ? 1 : std::min({seq->remaining(), budget, prefill_chunk_});
    const int new_len = seq->computed + count;
    bool keeps = true;
    while (cache_->reserve(id, new_len) != 1) {
      const int needed = pages_for(new_len, cache_->page_size());
      if (needed > num_pages_) {
        drop_running(id);
        cache_->release(id);
        failed->push_back({id, needed});
        sequences_.erase(id);
        keeps = false;
        break;
      }
      const int64_t victim = *std::max_element(running_.begin(), running_.end());   // the newest (engine.rs:632-639)
      planned->erase(std::remove_if(planned->begin(), planned->end(),
                                    [&](const PlannedEntry& p) { return p.id == victim; }), planned->end());
      Sequence* out = find(victim);
      drop_running(victim);
      cache_->release(victim);
      out->computed = 0;
      out->running = false;
      ++preemptions_;
      last_preempted_ = victim;
      preempted->push_back(victim);
      if (victim == id) { keeps = false; break; }
    }
    if (keeps) {
      planned->push_back({id, seq->computed, count, seq->computed + count == (int)seq->tokens.size()});
      budget -= count;
    }
  }
  // The budget of a preempted sequence's planned tokens is not handed out again in this iteration, as in the
  // reference's loop.  Oldest preempted sequence first, ahead of requests that never ran (engine.rs:369-376).
  std::vector<int64_t> back = *preempted;
  std::sort(back.begin(), back.end(), std::greater<int64_t>());
  for (int64_t id : back) waiting_.push_front(id);
}

int SchedulerCore::commit(int64_t id, int count) {
  Sequence* seq = find(id);
  if (!seq || !seq->running) return -1;
  seq->computed += count;
  if (seq->computed - count < seq->prompt_len)            // the portion held prompt tokens
    cache_->publish(id, seq->tokens.data(), seq->prompt_len);
  return 0;
}

int SchedulerCore::finish(int64_t id) {
  Sequence* seq = find(id);
  if (!seq) return -1;
  if (seq->running) {
    drop_running(id);
    cache_->release(id);
  } else {
    waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), id), waiting_.end());
  }
  sequences_.erase(id);
  return 0;
}

}  // namespace ta
