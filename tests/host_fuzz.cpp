// Drives the cache manager and the scheduler through their C entry points at random: requests of random lengths
// are added, cancelled and finished, every scheduled step is checked (starts equal cached lengths, the token budget
// holds, every slot lies inside its pool), some steps fail before they run, and the manager's audit must stay empty.
// Built with the address and undefined-behaviour sanitizers by tests/test_host_sanitized.py (host code only).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <random>
#include <string>
#include <vector>
extern "C" {
void* pa_cache_create(int, int, const int*, const int*, int);
void pa_cache_destroy(void*);
int pa_cache_open(void*, long long, int);
int pa_cache_reserve(void*, long long, int);
int pa_cache_commit(void*, long long, int);
int pa_cache_rollback(void*, long long);
int pa_cache_close(void*, long long);
int pa_cache_has(void*, long long);
int pa_cache_len(void*, long long);
int pa_cache_free_pages(void*, int);
int pa_cache_table(void*, long long, int, int*, int);
int pa_cache_fill_step(void*, int, const long long*, const int*, const int*, int, int*, int*, int*, int*, int*, int*, int*, int*);
const char* pa_cache_audit(void*);
int pa_cache_reservable_len(void*, long long);
void* pa_sched_create(void*, int, int, int, int, int, int, int);
void pa_sched_destroy(void*);
int pa_sched_add(void*, long long, int, int, int, int);
int pa_sched_schedule(void*, long long*, int*, int*, int*, int);
int pa_sched_step_done(void*);
void pa_sched_step_cancelled(void*);
int pa_sched_on_token(void*, long long);
int pa_sched_finish(void*, long long);
int pa_sched_num_waiting(void*);
int pa_sched_num_running(void*);
int pa_sched_info(void*, long long, int*);
int pa_sched_last_preempted(void*, long long*, int);
}
static void die(const char* what, unsigned seed, long it) { printf("FAIL %s (seed %u, iteration %ld)\n", what, seed, it); exit(1); }
int main(int argc, char** argv) {
  const unsigned seeds = argc > 1 ? atoi(argv[1]) : 50;
  long steps_total = 0, preempt = 0;
  for (unsigned seed = 0; seed < seeds; ++seed) {
    std::mt19937 rng(seed);
    auto R = [&](int lo, int hi) { return lo + (int)(rng() % (unsigned)(hi - lo + 1)); };
    const int page = 1 << R(0, 5);
    const int groups = R(1, 3);
    int pages[3], windows[3];
    for (int g = 0; g < groups; ++g) { pages[g] = R(0, 3) ? R(4, 40) : R(8, 200); windows[g] = R(0, 2) == 0 ? R(1, 300) : 0; }
    const int slots = R(0, 6);
    void* c = pa_cache_create(page, groups, pages, windows, slots);
    const int budget = R(4, 300);
    void* s = pa_sched_create(c, budget, R(0, 1) ? R(1, 100) : 0, R(1, 12), R(0, 1) ? R(50, 2000) : 0, R(0, 1) ? R(1, 200) : 0, R(0, 8), slots > 0 && R(0, 1));
    std::map<long long, int> left;   // new tokens still to come
    long long next_id = 1;
    for (long it = 0; it < 1500; ++it) {
      const int what = R(0, 9);
      if (what < 3 && left.size() < 20) {
        const int prompt = R(1, 200), mx = R(0, 2) ? R(1, 400) : R(1, 20);
        if (pa_sched_add(s, next_id, prompt, mx, R(0, 5) == 0, R(0, 3) == 0 ? R(1, 64) : 0) == 0) left[next_id] = mx;
        ++next_id;
      } else if (what == 3 && !left.empty()) {        // a request is cancelled from outside
        auto itx = left.begin(); std::advance(itx, R(0, (int)left.size() - 1));
        pa_sched_finish(s, itx->first); left.erase(itx);
      } else {
        long long ids[64]; int starts[64], counts[64], samples[64];
        const int n = pa_sched_schedule(s, ids, starts, counts, samples, 64);
        if (n < 0) die("more entries than running requests can be", seed, it);
        if (n == 0) continue;
        ++steps_total;
        int total = 0, stride = 1;
        for (int i = 0; i < n; ++i) {
          if (counts[i] < 1) die("an entry without tokens", seed, it);
          if (pa_cache_len(c, ids[i]) != starts[i]) die("start is not the cached length", seed, it);
          total += counts[i];
          const int need = (starts[i] + counts[i] + page - 1) / page;
          if (need > stride) stride = need;
        }
        if (total > budget) die("over the token budget", seed, it);
        std::vector<int> pos(total), sot(total), cu(n + 1), cl(n), ss(n), fr(n), bt((size_t)groups * n * stride), sl((size_t)groups * total);
        if (R(0, 7) == 0) { pa_sched_step_cancelled(s); }   // the step fails before it runs
        else {
          if (pa_cache_fill_step(c, n, ids, starts, counts, stride, pos.data(), sot.data(), cu.data(), cl.data(), ss.data(), fr.data(), bt.data(), sl.data()) != 0)
            die("fill_step refused a scheduled step", seed, it);
          for (int g = 0; g < groups; ++g)
            for (int t = 0; t < total; ++t) {
              const int v = sl[(size_t)g * total + t];
              if (v < -1 || v >= pages[g] * page) die("a slot outside the pool", seed, it);
            }
          if (pa_sched_step_done(s) != 0) die("step_done", seed, it);
          for (int i = 0; i < n; ++i)
            if (samples[i] && left.count(ids[i])) {
              if (--left[ids[i]] == 0 || R(0, 30) == 0) { pa_sched_finish(s, ids[i]); left.erase(ids[i]); }
              else if (pa_sched_on_token(s, ids[i]) != 0) die("on_token", seed, it);
            }
        }
        long long pre[64]; preempt += pa_sched_last_preempted(s, pre, 64);
      }
      const char* a = pa_cache_audit(c);
      if (a && a[0]) { printf("audit: %s\n", a); die("audit", seed, it); }
    }
    for (auto& kv : left) pa_sched_finish(s, kv.first);
    const char* a = pa_cache_audit(c);
    if (a && a[0]) { printf("audit at the end: %s\n", a); die("audit", seed, -1); }
    for (int g = 0; g < groups; ++g) if (pa_cache_free_pages(c, g) != pages[g]) die("pages lost", seed, -1);
    pa_sched_destroy(s); pa_cache_destroy(c);
  }
  printf("ok: %u seeds, %ld steps, %ld preemptions\n", seeds, steps_total, preempt);
  return 0;
}
