#include "scheduler.h"

#include <algorithm>
#include <climits>

namespace pa {

Scheduler::Scheduler(CacheManager* cache, const SchedulerConfig& cfg, bool needs_state)
    : cache_(cache), cfg_(cfg), needs_state_(needs_state) {
  if (cfg_.max_num_batched_tokens < 1) cfg_.max_num_batched_tokens = 1;
  if (cfg_.max_running_requests < 1) cfg_.max_running_requests = 1;
}

const Sequence* Scheduler::find(int64_t id) const {
  for (const auto& s : running_)
    if (s.id == id) return &s;
  for (const auto& s : waiting_)
    if (s.id == id) return &s;
  return nullptr;
}

int Scheduler::tokens_in_use() const {
  int t = 0;
  for (const auto& s : running_) t += s.known;
  return t;
}

bool Scheduler::add_request(int64_t id, int prompt_len, int max_new) {
  if (find(id) || cache_->has(id)) {
    error_ = "request " + std::to_string(id) + " is already live";
    return false;
  }
  if (prompt_len < 1) {
    error_ = "request " + std::to_string(id) + " has an empty prompt";
    return false;
  }
  if (max_new < 1) {
    error_ = "request " + std::to_string(id) + " asks for no new token";
    return false;
  }
  // Alone in an empty cache it must be able to run to its end.
  const int chunk_cap = cfg_.long_prefill_token_threshold > 0
                            ? std::min(cfg_.long_prefill_token_threshold, cfg_.max_num_batched_tokens)
                            : cfg_.max_num_batched_tokens;
  for (int g = 0; g < cache_->num_groups(); ++g) {
    const int need = cache_->peak_pages(prompt_len + max_new, chunk_cap, g);
    if (need > cache_->capacity_pages(g)) {
      error_ = "request " + std::to_string(id) + " needs " + std::to_string(need) + " pages of cache group " +
               std::to_string(g) + " for " + std::to_string(prompt_len) + " prompt and " + std::to_string(max_new) +
               " new tokens, the pool has " + std::to_string(cache_->capacity_pages(g));
      return false;
    }
  }
  if (needs_state_ && cache_->num_state_slots() < 1) {
    error_ = "the model keeps per-request state but the cache has no state slots";
    return false;
  }
  Sequence s;
  s.id = id;
  s.prompt_len = prompt_len;
  s.max_new = max_new;
  s.known = prompt_len;
  s.arrival = clock_++;
  waiting_.push_back(s);
  return true;
}

int Scheduler::chunk_for(const Sequence& s, int budget) const {
  int chunk = std::min(s.known - s.computed, budget);
  if (cfg_.long_prefill_token_threshold > 0) chunk = std::min(chunk, cfg_.long_prefill_token_threshold);
  return chunk;
}

int Scheduler::shrink_to_pages(const Sequence& s, int chunk) const {
  const int reach = cache_->reservable_len(s.id);
  return std::max(0, std::min(chunk, reach - s.computed));
}

bool Scheduler::tail_priority(const std::vector<StepEntry>& entries) const {
  const int threshold = cfg_.decode_priority_max_remaining_tokens;
  if (threshold <= 0) return false;
  bool any = false;
  for (const auto& e : entries) {
    const Sequence* s = find(e.id);
    if (!s || s->generated == 0 || e.count != 1 || !e.samples) continue;  // not a decoding request
    any = true;
    if (s->remaining() > threshold) return false;
  }
  return any;
}

void Scheduler::preempt(size_t idx) {
  Sequence s = running_[idx];
  running_.erase(running_.begin() + idx);
  cache_->close(s.id);
  s.computed = 0;
  s.preempt_count += 1;
  waiting_.push_front(s);
  last_preempted_.push_back(s.id);
  preemptions_ += 1;
}

bool Scheduler::enforce_token_cap() {
  if (cfg_.max_total_tokens <= 0) return false;
  bool any = false;
  // every running request may grow by one token this step
  while (running_.size() > 1 && tokens_in_use() + (int)running_.size() > cfg_.max_total_tokens) {
    size_t newest = 0;
    for (size_t i = 1; i < running_.size(); ++i)
      if (running_[i].arrival > running_[newest].arrival) newest = i;
    preempt(newest);
    any = true;
  }
  return any;
}

void Scheduler::admit_waiting(int& budget) {
  const int G = cache_->num_groups();
  const int chunk_cap = cfg_.long_prefill_token_threshold > 0
                            ? std::min(cfg_.long_prefill_token_threshold, cfg_.max_num_batched_tokens)
                            : cfg_.max_num_batched_tokens;
  // Pages that running requests will still take for tokens they already know
  // of (unfinished prompts): not free for newcomers.
  std::vector<int> owed(G, 0);
  for (const auto& s : running_) {
    const RequestCache* rc = cache_->find(s.id);
    if (!rc || rc->reserved_len >= s.known) continue;
    for (int g = 0; g < G; ++g)
      owed[g] += std::max(0, cache_->peak_pages(s.known, chunk_cap, g) - cache_->live_pages(s.id, g));
  }
  while (!waiting_.empty() && (int)running_.size() < cfg_.max_running_requests && budget > 0) {
    Sequence& s = waiting_.front();
    if (needs_state_ && cache_->free_state_slots() == 0) break;
    if (cfg_.max_total_tokens > 0 && !running_.empty() && tokens_in_use() + s.known + 1 > cfg_.max_total_tokens) break;
    const int total = s.known + std::min(std::max(0, s.remaining()), cfg_.decode_reservation_cap);
    std::vector<int> need(G);
    bool fits = true;
    for (int g = 0; g < G; ++g) {
      need[g] = cache_->peak_pages(total, chunk_cap, g);
      if (need[g] + owed[g] > cache_->free_pages(g)) fits = false;
    }
    if (!fits) break;
    const int chunk = chunk_for(s, budget);
    if (chunk < 1) break;
    if (!cache_->open(s.id, needs_state_)) break;
    if (cache_->reserve(s.id, chunk) != 0) {  // cannot happen after the test above
      cache_->close(s.id);
      break;
    }
    step_.push_back(StepEntry{s.id, 0, chunk, chunk == s.known ? 1 : 0});
    budget -= chunk;
    for (int g = 0; g < G; ++g) owed[g] += std::max(0, need[g] - cache_->live_pages(s.id, g));
    running_.push_back(s);
    waiting_.pop_front();
  }
}

const std::vector<StepEntry>& Scheduler::schedule() {
  step_.clear();
  last_preempted_.clear();
  error_.clear();
  bool had_preemption = enforce_token_cap();
  for (;;) {
    int budget = cfg_.max_num_batched_tokens;
    bool blocked = false;
    for (auto& s : running_) {
      if (budget == 0) break;
      int chunk = shrink_to_pages(s, chunk_for(s, budget));
      if (chunk < 1) {
        blocked = true;
        continue;
      }
      if (cache_->reserve(s.id, s.computed + chunk) != 0) {
        blocked = true;
        continue;
      }
      step_.push_back(StepEntry{s.id, s.computed, chunk, s.computed + chunk == s.known ? 1 : 0});
      budget -= chunk;
    }
    if (!had_preemption && !blocked && budget > 0 && !tail_priority(step_)) admit_waiting(budget);
    if (!step_.empty() || running_.empty()) break;
    // No request can move: every running one waits for a page.
    if (running_.size() <= 1) {
      error_ = "request " + std::to_string(running_[0].id) + " cannot get a page although it runs alone";
      break;
    }
    size_t oldest = 0;
    for (size_t i = 1; i < running_.size(); ++i)
      if (running_[i].arrival < running_[oldest].arrival) oldest = i;
    size_t victim = SIZE_MAX;
    for (size_t i = 0; i < running_.size(); ++i) {
      if (i == oldest) continue;
      if (victim == SIZE_MAX || running_[i].preempt_count > running_[victim].preempt_count ||
          (running_[i].preempt_count == running_[victim].preempt_count &&
           running_[i].arrival > running_[victim].arrival))
        victim = i;
    }
    preempt(victim);
    had_preemption = true;
  }
  return step_;
}

bool Scheduler::step_done() {
  for (const auto& e : step_) {
    if (!cache_->commit(e.id, e.start + e.count)) {
      error_ = cache_->error();
      return false;
    }
    for (auto& s : running_)
      if (s.id == e.id) s.computed = e.start + e.count;
  }
  step_.clear();
  return true;
}

void Scheduler::step_cancelled() {
  for (const auto& e : step_) cache_->rollback(e.id);
  step_.clear();
}

bool Scheduler::on_token(int64_t id) {
  for (auto& s : running_) {
    if (s.id != id) continue;
    if (s.computed != s.known) {
      error_ = "request " + std::to_string(id) + " got a token before its known tokens were all fed";
      return false;
    }
    s.known += 1;
    s.generated += 1;
    return true;
  }
  error_ = "request " + std::to_string(id) + " is not running";
  return false;
}

bool Scheduler::finish(int64_t id) {
  for (size_t i = 0; i < running_.size(); ++i) {
    if (running_[i].id != id) continue;
    step_.erase(std::remove_if(step_.begin(), step_.end(), [&](const StepEntry& e) { return e.id == id; }),
                step_.end());
    cache_->close(id);
    running_.erase(running_.begin() + i);
    return true;
  }
  for (size_t i = 0; i < waiting_.size(); ++i) {
    if (waiting_[i].id != id) continue;
    waiting_.erase(waiting_.begin() + i);
    return true;
  }
  error_ = "request " + std::to_string(id) + " is unknown";
  return false;
}

}  // namespace pa
