// C entry points of the host runtime (cache manager and scheduler) for the
// Python side.  Handles are opaque pointers; strings returned stay valid until
// the next call on the same handle.
#include <cstring>
#include <vector>

#include "cache_manager.h"
#include "scheduler.h"

using pa::CacheManager;
using pa::Scheduler;

namespace {
struct CacheHandle {
  CacheManager mgr;
  std::string text;
  CacheHandle(int page_size, const std::vector<pa::GroupSpec>& groups, int slots) : mgr(page_size, groups, slots) {}
};
struct SchedHandle {
  Scheduler sched;
  SchedHandle(CacheManager* c, const pa::SchedulerConfig& cfg, bool st) : sched(c, cfg, st) {}
};
}  // namespace

extern "C" {

void* pa_cache_create(int page_size, int n_groups, const int* num_pages, const int* windows, int state_slots) {
  if (page_size < 1 || n_groups < 0) return nullptr;
  std::vector<pa::GroupSpec> groups(n_groups);
  for (int g = 0; g < n_groups; ++g) {
    groups[g].num_pages = num_pages[g];
    groups[g].window = windows[g];
  }
  return new CacheHandle(page_size, groups, state_slots);
}
void pa_cache_destroy(void* h) { delete static_cast<CacheHandle*>(h); }
static CacheManager& M(void* h) { return static_cast<CacheHandle*>(h)->mgr; }

int pa_cache_open(void* h, long long id, int need_state) { return M(h).open(id, need_state != 0) ? 0 : -1; }
int pa_cache_reserve(void* h, long long id, int new_len) { return M(h).reserve(id, new_len); }
int pa_cache_commit(void* h, long long id, int new_len) { return M(h).commit(id, new_len) ? 0 : -1; }
int pa_cache_rollback(void* h, long long id) { return M(h).rollback(id) ? 0 : -1; }
int pa_cache_close(void* h, long long id) { return M(h).close(id) ? 0 : -1; }
int pa_cache_has(void* h, long long id) { return M(h).has(id) ? 1 : 0; }
int pa_cache_len(void* h, long long id) {
  const pa::RequestCache* rc = M(h).find(id);
  return rc ? rc->len : -1;
}
int pa_cache_state_slot(void* h, long long id) {
  const pa::RequestCache* rc = M(h).find(id);
  return rc ? rc->state_slot : -1;
}
int pa_cache_page_size(void* h) { return M(h).page_size(); }
int pa_cache_num_groups(void* h) { return M(h).num_groups(); }
int pa_cache_free_pages(void* h, int g) { return M(h).free_pages(g); }
int pa_cache_capacity_pages(void* h, int g) { return M(h).capacity_pages(g); }
int pa_cache_free_state_slots(void* h) { return M(h).free_state_slots(); }
int pa_cache_num_requests(void* h) { return M(h).num_requests(); }
int pa_cache_live_pages(void* h, long long id, int g) { return M(h).live_pages(id, g); }
int pa_cache_reservable_len(void* h, long long id) { return M(h).reservable_len(id); }
int pa_cache_peak_pages(void* h, int total, int chunk, int g) { return M(h).peak_pages(total, chunk, g); }
// Copies the table of group g (logical page -> physical page, -1 = given back); returns its length.
int pa_cache_table(void* h, long long id, int g, int* out, int cap) {
  const pa::RequestCache* rc = M(h).find(id);
  if (!rc || g < 0 || g >= M(h).num_groups()) return -1;
  const auto& t = rc->tables[g];
  for (int i = 0; i < (int)t.size() && i < cap; ++i) out[i] = t[i];
  return (int)t.size();
}
int pa_cache_fill_step(void* h, int n, const long long* ids, const int* starts, const int* counts, int table_stride,
                       int* positions, int* seq_of_token, int* cu_q, int* context_lens, int* state_slots, int* fresh,
                       int* block_tables, int* slots) {
  static_assert(sizeof(long long) == sizeof(int64_t), "id width");
  return M(h).fill_step(n, reinterpret_cast<const int64_t*>(ids), starts, counts, table_stride, positions, seq_of_token,
                        cu_q, context_lens, state_slots, fresh, block_tables, slots)
             ? 0
             : -1;
}
const char* pa_cache_audit(void* h) {
  auto* ch = static_cast<CacheHandle*>(h);
  ch->text = ch->mgr.audit();
  return ch->text.c_str();
}
const char* pa_cache_error(void* h) { return M(h).error().c_str(); }

void* pa_sched_create(void* cache, int max_num_batched_tokens, int long_prefill_token_threshold,
                      int max_running_requests, int max_total_tokens, int decode_reservation_cap,
                      int decode_priority_max_remaining_tokens, int needs_state) {
  pa::SchedulerConfig cfg;
  cfg.max_num_batched_tokens = max_num_batched_tokens;
  cfg.long_prefill_token_threshold = long_prefill_token_threshold;
  cfg.max_running_requests = max_running_requests;
  cfg.max_total_tokens = max_total_tokens;
  cfg.decode_reservation_cap = decode_reservation_cap;
  cfg.decode_priority_max_remaining_tokens = decode_priority_max_remaining_tokens;
  return new SchedHandle(&M(cache), cfg, needs_state != 0);
}
void pa_sched_destroy(void* h) { delete static_cast<SchedHandle*>(h); }
static Scheduler& S(void* h) { return static_cast<SchedHandle*>(h)->sched; }

int pa_sched_add(void* h, long long id, int prompt_len, int max_new, int atomic, int max_chunk) {
  return S(h).add_request(id, prompt_len, max_new, atomic != 0, max_chunk) ? 0 : -1;
}
// Decides a step; writes up to cap entries and returns their number (or -1 if cap is too small).
int pa_sched_schedule(void* h, long long* ids, int* starts, int* counts, int* samples, int cap) {
  const auto& step = S(h).schedule();
  if ((int)step.size() > cap) {
    S(h).step_cancelled();
    return -1;
  }
  for (size_t i = 0; i < step.size(); ++i) {
    ids[i] = step[i].id;
    starts[i] = step[i].start;
    counts[i] = step[i].count;
    samples[i] = step[i].samples;
  }
  return (int)step.size();
}
int pa_sched_step_done(void* h) { return S(h).step_done() ? 0 : -1; }
void pa_sched_step_cancelled(void* h) { S(h).step_cancelled(); }
int pa_sched_on_token(void* h, long long id) { return S(h).on_token(id) ? 0 : -1; }
int pa_sched_finish(void* h, long long id) { return S(h).finish(id) ? 0 : -1; }
int pa_sched_num_waiting(void* h) { return S(h).num_waiting(); }
int pa_sched_num_running(void* h) { return S(h).num_running(); }
int pa_sched_tokens_in_use(void* h) { return S(h).tokens_in_use(); }
long pa_sched_preemptions(void* h) { return S(h).preemptions(); }
int pa_sched_last_preempted(void* h, long long* out, int cap) {
  const auto& v = S(h).last_preempted();
  for (size_t i = 0; i < v.size() && (int)i < cap; ++i) out[i] = v[i];
  return (int)v.size();
}
// Fields of a request: known, computed, generated, max_new, preempt_count, running(1)/waiting(0). Returns -1 if unknown.
int pa_sched_info(void* h, long long id, int* out6) {
  const pa::Sequence* s = S(h).find(id);
  if (!s) return -1;
  out6[0] = s->known;
  out6[1] = s->computed;
  out6[2] = s->generated;
  out6[3] = s->max_new;
  out6[4] = s->preempt_count;
  out6[5] = S(h).is_running(id) ? 1 : 0;
  return 0;
}
const char* pa_sched_error(void* h) { return S(h).error().c_str(); }

}  // extern "C"
