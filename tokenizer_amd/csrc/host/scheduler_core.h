// The scheduler's decisions: a FIFO of waiting sequences and a running batch above the cache manager.
// Policy follows qwen-server/src/engine.rs: admission looks at the front of the queue only and reserves pages
// for the whole prompt (458-517); each iteration grows the running sequences oldest first and, when pages run
// out, preempts the newest one, which gives back everything and is recomputed later (561-668); preempted
// sequences return to the front of the queue, oldest first (369-376); a sequence that cannot fit in the whole
// pool fails (473-487, 670-685).  Beyond the reference one iteration is a single mixed batch under a token
// budget: one token for every decoding sequence first, then portions of prompts in order of arrival; or, with
// `prompts_first`, in the reference's order within an iteration (new sequences are prefilled before the batched
// decode, 788-805), which under a budget means more than an order: portions of prompts take the budget first and
// decoding sequences what is left of it, so that they wait while prompts stand in line and then decode together
// (the reference has no budget: there every decoding sequence still gets its token in the same iteration).
// Sampling, stop conditions and results stay with the caller; this class owns the token lists, the order of
// work and every exchange with the cache manager.
#pragma once
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache_core.h"

namespace ta {

struct Sequence {
  int64_t id = 0;
  int prompt_len = 0;
  std::vector<int32_t> tokens;       // the prompt and every sampled id that is to be forwarded
  int computed = 0;                  // tokens whose keys and values are in the cache
  bool running = false;
  int sampled() const { return (int)tokens.size() - prompt_len; }
  int remaining() const { return (int)tokens.size() - computed; }
  bool decoding() const { return sampled() > 0 && remaining() == 1; }
};

struct PlannedEntry { int64_t id; int first, count; bool completes; };   // tokens [first, first + count) of the sequence
struct FailedEntry { int64_t id; int pages_needed; };

class SchedulerCore {
 public:
  SchedulerCore(CacheCore* cache, int num_pages, int max_batch_size, int token_budget, int prefill_chunk,
                bool prompts_first = false);

  int enqueue(int64_t id, const int32_t* prompt, int count);   // 0, or -1 if the id is known
  int append_token(int64_t id, int32_t token);
  const Sequence* find(int64_t id) const;
  int n_running() const { return (int)running_.size(); }
  int n_waiting() const { return (int)waiting_.size(); }
  int max_running() const { return max_running_; }
  int preemptions() const { return preemptions_; }
  int64_t last_preempted_id() const { return last_preempted_; }
  int prefix_hits() const { return prefix_hits_; }                   // admissions that found shared pages
  int64_t prefix_tokens_reused() const { return prefix_tokens_; }    // tokens those pages held
  int64_t front_waiting() const { return waiting_.empty() ? -1 : waiting_.front(); }
  int pages_to_admit(int64_t id) const;
  const std::vector<int64_t>& running() const { return running_; }
  const std::deque<int64_t>& waiting() const { return waiting_; }

  // One iteration's decisions: admission, then the plan (pages reserved), then the preempted back to the queue.
  void plan_step(std::vector<PlannedEntry>* planned, std::vector<int64_t>* preempted, std::vector<FailedEntry>* failed);
  // The step ran `count` more tokens of the sequence: they are in the cache now; full prompt pages become shareable.
  int commit(int64_t id, int count);
  // The sequence is over (finished, cancelled or failed by the caller): everything it holds goes back.
  int finish(int64_t id);

 private:
  Sequence* find(int64_t id);
  void admit(std::vector<FailedEntry>* failed);
  void drop_running(int64_t id);

  CacheCore* cache_;
  int num_pages_, max_batch_size_, token_budget_, prefill_chunk_;
  bool prompts_first_;
  std::unordered_map<int64_t, Sequence> sequences_;
  std::deque<int64_t> waiting_;
  std::vector<int64_t> running_;          // in order of admission
  int max_running_ = 0, preemptions_ = 0, prefix_hits_ = 0;
  int64_t prefix_tokens_ = 0;
  int64_t last_preempted_ = 0;
};

}  // namespace ta
