// CPU test of BatchScheduler (csrc/kv_batcher.hpp): the bookkeeping of the continuous-batching driver, no GPU call.
// Random workloads over many seeds and pool sizes; after every Schedule and every Commit the invariants a page table
// lives by are checked from outside: every page has exactly one holder or is free, a request holds exactly the pages
// its length needs (its planned work included), work continues where the request stands, the limits hold, requests
// are admitted in the order they came (a request put back goes first), and every request ends.
#include <cstdio>
#include <map>
#include <random>
#include <set>
#include <vector>

#include "kv_batcher.hpp"

using namespace yahkv_host;

namespace {

struct Fail : std::runtime_error {
  using std::runtime_error::runtime_error;
};
void Expect(bool ok, const char* what) {
  if (!ok) throw Fail(what);
}
template <typename F>
void ExpectThrow(F&& f, const char* what) {
  try {
    f();
  } catch (const KvError&) {
    return;
  }
  throw Fail(what);
}

struct Spec {
  int prompt, max_new;
};

// One random workload; returns the number of requests put back.
int64_t RunOne(uint32_t seed) {
  std::mt19937 rng(seed);
  const int pt = 1 << (4 + rng() % 3);                      // 16, 32, 64
  const int context = pt * int(2 + rng() % 12);
  const int chunk = int(1 + rng() % (2 * pt));
  const int max_running = int(1 + rng() % 8), max_prefill = int(1 + rng() % max_running);
  const int ctx_pages = context / pt;
  const int n_pages = ctx_pages + int(rng() % (3 * ctx_pages + 1));  // from "one request fits" to roomy
  BatchScheduler b(n_pages, pt, max_running, context, chunk, max_prefill, rng() % 2 ? seed + 1 : 0);
  const int n_req = int(1 + rng() % 40);
  std::map<int64_t, Spec> spec;
  std::map<int64_t, int> stands;      // positions done, as this test counts them
  std::vector<int64_t> order;         // ids in the order they must be admitted
  std::set<int64_t> admitted;
  int64_t next_id = 1;
  int submitted = 0, finished = 0;
  auto submit = [&] {
    Spec s{int(1 + rng() % context), 0};
    s.max_new = int(rng() % (context - s.prompt + 1));
    spec[next_id] = s, stands[next_id] = 0;
    b.Submit(next_id, s.prompt, s.max_new);
    order.push_back(next_id);
    ++next_id, ++submitted;
  };
  auto check_pages = [&](const BatchPlan* plan) {
    std::set<int32_t> seen;
    int held = 0;
    for (int64_t id : b.holders()) {
      const std::vector<int32_t>& pg = b.pages(id);
      for (int32_t p : pg) {
        Expect(p >= 0 && p < n_pages, "page id in range");
        Expect(seen.insert(p).second, "a page has one holder");
        Expect(b.pool().owners(p) == 1, "a held page has one owner in the allocator");
      }
      held += int(pg.size());
      int need = b.length(id);  // tokens the pages must cover: what is done plus what is planned
      if (plan != nullptr)
        for (const auto* list : {&plan->prefill, &plan->decode})
          for (const BatchWork& w : *list)
            if (w.id == id) need = w.pos + w.n;
      Expect(int(pg.size()) == (need + pt - 1) / pt, "a request holds the pages its length needs, no more");
    }
    Expect(held + b.free_pages() == n_pages, "held and free pages add up to the pool");
  };
  for (int i = int(rng() % 4); i > 0 && submitted < n_req; --i) submit();
  int steps = 0, idle_steps = 0;
  while (submitted < n_req || !b.idle()) {
    if (submitted < n_req && rng() % 3 == 0) submit();
    Expect(++steps < 100000, "the scheduler makes no progress");
    const int64_t put_back_before = b.stats().preempted;
    const std::vector<int64_t> running_before = b.holders();
    const BatchPlan plan = b.Schedule();
    ExpectThrow([&] { b.Schedule(); }, "Schedule twice must throw");
    Expect(int(plan.prefill.size()) <= max_prefill && b.running() <= max_running, "limits");
    std::set<int64_t> in_plan;
    for (const auto* list : {&plan.prefill, &plan.decode})
      for (const BatchWork& w : *list) {
        Expect(in_plan.insert(w.id).second, "one piece of work per request and step");
        const Spec& s = spec.at(w.id);
        if (w.pos == 0 && stands[w.id] != 0) stands[w.id] = 0;  // put back and started again
        Expect(w.pos == stands[w.id], "work continues where the request stands");
        const bool pre = list == &plan.prefill;
        Expect(pre ? (w.pos < s.prompt && w.n == std::min(chunk, s.prompt - w.pos)) : (w.pos >= s.prompt && w.n == 1),
               "prompt chunks before decode tokens, of the right size");
        Expect(w.pos + w.n <= s.prompt + s.max_new || (pre && s.max_new == 0), "work within the request");
      }
    // admissions follow the queue: newly running ids are the head of `order`
    for (int64_t id : b.holders()) {
      if (admitted.count(id)) continue;
      Expect(!order.empty() && order.front() == id, "requests are admitted in the order they came");
      order.erase(order.begin());
      admitted.insert(id);
    }
    // a request put back is queued again, at the head, in the order in which they were admitted
    if (b.stats().preempted > put_back_before) {
      const std::vector<int64_t> now = b.holders();
      std::vector<int64_t> back;
      for (int64_t id : running_before)
        if (std::find(now.begin(), now.end(), id) == now.end() && spec.count(id)) back.push_back(id);
      for (auto it = back.rbegin(); it != back.rend(); ++it) order.insert(order.begin(), *it), admitted.erase(*it), stands[*it] = 0;
      const std::vector<int64_t> waiting = b.waiting();
      Expect(waiting.size() >= back.size() && std::equal(back.begin(), back.end(), waiting.begin()),
             "requests put back wait at the head of the queue");
    }
    check_pages(&plan);
    idle_steps = plan.empty() ? idle_steps + 1 : 0;
    Expect(idle_steps < 3 || b.idle(), "a step with waiting requests plans some work");
    b.Commit();
    for (const auto* list : {&plan.prefill, &plan.decode})
      for (const BatchWork& w : *list) stands[w.id] = w.pos + w.n;
    check_pages(nullptr);
    if (rng() % 50 == 0 && !b.holders().empty()) {  // a client goes away
      const std::vector<int64_t> h = b.holders();
      b.Stop(h[rng() % h.size()]);
    }
    for (int64_t id : b.TakeFinished()) {
      Expect(spec.count(id) == 1, "a request ends once");
      spec.erase(id), stands.erase(id), admitted.erase(id);
      ++finished;
    }
  }
  Expect(finished == n_req && b.free_pages() == n_pages, "every request ends and every page is free again");
  Expect(b.stats().admitted == n_req + b.stats().preempted, "every request put back is admitted again");
  return b.stats().preempted;
}

}  // namespace

int main(int argc, char** argv) {
  try {
    const int n = argc > 1 ? std::atoi(argv[1]) : 400;
    int64_t put_back = 0;
    for (int seed = 1; seed <= n; ++seed) {
      try {
        put_back += RunOne(uint32_t(seed));
      } catch (const std::exception& e) {
        std::fprintf(stderr, "kv_scheduler_test: FAILED at seed %d: %s\n", seed, e.what());
        return 1;
      }
    }
    ExpectThrow([] { BatchScheduler b(8, 16, 2, 64, 16, 3); }, "more chunks per step than running requests must be refused");
    ExpectThrow([] { BatchScheduler b(8, 16, 2, 64, 16, 1); b.Commit(); }, "Commit without Schedule must throw");
    Expect(put_back > 0, "some workload was meant to run out of pages");
    std::printf("kv_scheduler_test: ok (%d workloads, %lld requests put back)\n", n, (long long)put_back);
    return 0;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "kv_scheduler_test: FAILED: %s\n", e.what());
    return 1;
  }
}
