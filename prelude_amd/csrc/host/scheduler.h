// Continuous batching with chunked prefill under one token budget per step.
//
// The decisions follow the reference's chunked-prefill mode
// (crates/prelude-core/src/scheduler/admission.rs:101-194 running requests
// first, then waiting ones first-come first-served; :297-428 admission by
// pages with the growth owed to running prefills held back; :431-469 chunk
// size; crates/prelude-core/src/scheduler/preemption.rs:50-116 who is evicted;
// crates/prelude-core/src/scheduler/state.rs:224-243 the knobs and defaults).
//
// Ours: a request is a run of known tokens of which `computed` have their
// keys cached; every step feeds known[computed : computed + chunk], and a
// token is sampled exactly when the chunk reaches the end of what is known.
// Decoding is the case chunk == 1.  An evicted request therefore recomputes
// prompt and generated tokens alike (the reference re-feeds the prompt only,
// crates/prelude-core/src/scheduler/preemption.rs:7-27).  When pages run out:
// a running request's portion is shortened to the pages that are left, or
// skipped for this step; if no request at all can move, the one evicted most
// often (then the newest) other than the oldest goes back to the front of the
// waiting queue with nothing cached, at once rather than after 16 idle steps
// (crates/prelude-core/src/engine/run/ar.rs:202-203, :305-327), because
// nothing else can change between two steps of a synchronous loop.
#pragma once
#include <cstdint>
#include <deque>
#include <string>
#include <vector>

#include "cache_manager.h"

namespace pa {

struct SchedulerConfig {
  int max_num_batched_tokens = 8192;       // tokens per step, prompt portions and decode tokens together
  int long_prefill_token_threshold = 0;    // cap on one request's portion; 0 = none
  int max_running_requests = 256;
  int max_total_tokens = 0;                // cap on tokens held by running requests; 0 = pages decide alone
  int decode_reservation_cap = 4096;       // future tokens reserved per request at admission
  int decode_priority_max_remaining_tokens = 4;
};

struct StepEntry {
  int64_t id;
  int start;    // first position fed
  int count;    // tokens fed
  int samples;  // 1 when the last fed token is the last known one: its logits give the next token
};

struct Sequence {
  int64_t id = 0;
  int prompt_len = 0;
  int max_new = 0;
  int known = 0;      // prompt + generated tokens
  int computed = 0;   // tokens whose keys are cached
  int generated = 0;
  uint64_t arrival = 0;
  int preempt_count = 0;
  bool finished = false;
  // A request whose mixers cannot continue a prompt from a cut (their state does not carry across portions):
  // what it still has to feed is fed whole in one step or not at all.  Single decode tokens are not meant.
  bool atomic = false;
  int max_chunk = 0;  // cap on this request's portion (0 = none), beside the scheduler's own
  int remaining() const { return max_new - generated; }
};

class Scheduler {
 public:
  Scheduler(CacheManager* cache, const SchedulerConfig& cfg, bool needs_state);

  const SchedulerConfig& config() const { return cfg_; }
  // False (with error()) if the id is in use, the prompt is empty, or the
  // request could never fit the cache (or, fed whole, the step's token budget) even alone.
  // `atomic`: feed what is known whole or not at all; `max_chunk`: cap on its portions, 0 = none.
  bool add_request(int64_t id, int prompt_len, int max_new, bool atomic = false, int max_chunk = 0);
  // Decides one step and reserves its pages.  Empty when nothing can run.
  const std::vector<StepEntry>& schedule();
  // The step just scheduled has run: what it fed is cached now.
  bool step_done();
  // The step just scheduled will not run: give its pages back.
  void step_cancelled();
  // A token was sampled for a request whose last entry had samples == 1.
  bool on_token(int64_t id);
  // The request is over (any reason): its pages and slot go back.
  bool finish(int64_t id);

  int num_waiting() const { return (int)waiting_.size(); }
  int num_running() const { return (int)running_.size(); }
  int tokens_in_use() const;
  long preemptions() const { return preemptions_; }
  // Requests evicted by the last schedule() (they restart from nothing).
  const std::vector<int64_t>& last_preempted() const { return last_preempted_; }
  const Sequence* find(int64_t id) const;
  bool is_running(int64_t id) const {
    for (const auto& s : running_)
      if (s.id == id) return true;
    return false;
  }
  const std::string& error() const { return error_; }

 private:
  int chunk_for(const Sequence& s, int budget) const;
  int shrink_to_pages(const Sequence& s, int chunk) const;
  int portion_for(const Sequence& s, int budget) const;
  bool tail_priority(const std::vector<StepEntry>& entries) const;
  void admit_waiting(int& budget);
  void preempt(size_t idx);
  bool enforce_token_cap();

  CacheManager* cache_;
  SchedulerConfig cfg_;
  bool needs_state_;
  std::deque<Sequence> waiting_;
  std::vector<Sequence> running_;
  std::vector<StepEntry> step_;
  std::vector<int64_t> last_preempted_;
  uint64_t clock_ = 0;
  long preemptions_ = 0;
  std::string error_;
};

}  // namespace pa
