// GPU test of the continuous-batching driver (csrc/kv_batcher.hpp) against the CPU oracle. Twelve requests with prompts
// of 5 to 150 tokens and 0 to 40 generated tokens go through a pool that is too small to hold them all, so requests
// wait, run next to each other, are put back and start again; two layers share the page table. Every row is a
// function of (layer, request, position) alone; the oracle keeps each request's layer in a pool of its own with an
// identity page table, so whatever the batcher does with
// pages and batches must not show in the numbers: every attention output within 2e-3 of the oracle's, every
// request's blocks bit-exact when it ends, and all pages free again at the end.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <random>
#include <vector>

#include "kv_batcher.hpp"
#include "yahkv_oracle.h"

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

constexpr int NQ = 8, H = 2, D = 128, PT = 16, T = 192, CHUNK = 32, LAYERS = 2;

// Row `kind` (0 K, 1 V, 2 Q) of (layer, request, position): bf16 normals from a generator seeded by the triple.
void Row(int layer, int64_t id, int pos, int kind, int n, uint16_t* bits, float* f) {
  std::mt19937 rng(uint32_t(id * 7919 + pos * 31 + kind * 1000003 + layer * 50021 + 17));
  std::normal_distribution<float> nd;
  for (int i = 0; i < n; ++i) {
    bits[i] = orc_f32_to_bf16(nd(rng));
    if (f != nullptr) f[i] = orc_bf16_to_f32(bits[i]);
  }
}

// One layer of one request in the oracle: a pool of its own, identity page table.
struct Mirror {
  orc_geometry og{8, NQ, H, D, PT, T / PT};
  std::vector<uint8_t> kq, vq;
  std::vector<uint16_t> ks, vs;
  std::vector<int32_t> table;
  int done = 0;
  Mirror() : kq(orc_kq_bytes(&og), 0), vq(orc_vq_bytes(&og), 0), ks(orc_ks_bytes(&og) / 2, 0), vs(orc_vs_bytes(&og) / 2, 0) {
    for (int p = 0; p < T / PT; ++p) table.push_back(p);
  }
  orc_pools pools() { return orc_pools{kq.data(), ks.data(), vq.data(), vs.data()}; }
};

double RelErr(const float* got, const float* want, size_t n) {
  double d = 0, m = 0;
  for (size_t i = 0; i < n; ++i) d = std::max(d, std::fabs(double(got[i]) - want[i])), m = std::max(m, std::fabs(double(want[i])));
  return d / m;
}

}  // namespace

namespace {
int RunTest() {
  try {
    const int n_pages = 26;  // 416 tokens: about three of the longer requests
    const yahkv_geometry g{YAHKV_Q8_0, NQ, H, D, PT, n_pages};
    const int max_running = 5, max_prefill = 2;
    KvBatcher b(g, LAYERS, max_running, T, CHUNK, max_prefill, nullptr, /*shuffle_seed=*/5);
    ExpectThrow([&] { b.Submit(1, 0, 4); }, "an empty prompt must be refused");
    ExpectThrow([&] { b.Submit(1, T, 1); }, "a request past the context must be refused");
    ExpectThrow([&] { b.RunLayer(0, nullptr, nullptr, nullptr, nullptr, YAHKV_F32, nullptr, nullptr, nullptr, YAHKV_BF16, nullptr, YAHKV_BF16, 1.0f); },
                "RunLayer without Schedule must throw");
    ExpectThrow([&] { b.Commit(); }, "Commit without Schedule must throw");

    std::mt19937 rng(11);
    struct Spec { int prompt, max_new; };
    std::map<int64_t, Spec> spec;
    std::map<int64_t, std::vector<Mirror>> mirror;
    std::map<int64_t, int> outputs;  // attention rows checked per request
    const int n_req = 12;
    for (int64_t id = 100; id < 100 + n_req; ++id) {
      Spec s{int(5 + rng() % 146), int(rng() % 41)};
      if (id == 103) s = Spec{150, 40};  // a long one
      if (id == 105) s = Spec{33, 0};    // ends with its prompt
      spec[id] = s;
    }
    ExpectThrow([&] { KvBatcher tiny(yahkv_geometry{YAHKV_Q8_0, NQ, H, D, PT, 4}, 1, 2, T, CHUNK, 1); tiny.Submit(1, 100, 0); },
                "a request larger than the pool must be refused");

    const size_t kv_row = size_t(H) * D, q_row = size_t(NQ) * D;
    DeviceBuffer pk(max_prefill * CHUNK * kv_row * 2), pv(max_prefill * CHUNK * kv_row * 2), pq(max_prefill * CHUNK * q_row * 2);
    DeviceBuffer pout(max_prefill * CHUNK * q_row * 4);
    DeviceBuffer dk(max_running * kv_row * 2), dv(max_running * kv_row * 2), dq(max_running * q_row * 2), dout(max_running * q_row * 4);
    std::vector<uint16_t> hk, hv, hq;
    const float scale = 1.0f / std::sqrt(float(D));
    double worst = 0;
    int64_t next_submit = 100;
    int steps = 0;
    // arrivals: four at once, then one more every other step
    auto arrive = [&](int n) {
      for (; n > 0 && next_submit < 100 + n_req; --n, ++next_submit) {
        b.Submit(next_submit, spec[next_submit].prompt, spec[next_submit].max_new);
        mirror.emplace(next_submit, std::vector<Mirror>(LAYERS));
      }
    };
    arrive(4);
    ExpectThrow([&] { b.Submit(100, 5, 5); }, "a request id in use must be refused");
    while (!b.idle() || next_submit < 100 + n_req) {
      if (steps % 2 == 1) arrive(1);
      Expect(++steps < 2000, "the batcher makes no progress");
      const BatchPlan plan = b.Schedule();
      ExpectThrow([&] { b.Schedule(); }, "Schedule twice must throw");
      const int np = int(plan.prefill.size()), nd = int(plan.decode.size());
      Expect(np <= max_prefill && np + nd <= max_running + max_prefill && b.running() <= max_running, "plan within the limits");
      // a request that was put back starts again from its first token
      for (const auto& list : {plan.prefill, plan.decode})
        for (const BatchWork& w : list) {
          std::vector<Mirror>& m = mirror.at(w.id);
          if (w.pos == 0 && m[0].done != 0) m = std::vector<Mirror>(LAYERS), outputs[w.id] = 0;
          Expect(w.pos == m[0].done, "work continues where the request stands");
        }
      ExpectThrow([&] { b.RunLayer(LAYERS, nullptr, nullptr, nullptr, nullptr, YAHKV_F32, nullptr, nullptr, nullptr, YAHKV_BF16, nullptr, YAHKV_BF16, 1.0f); },
                  "a layer that does not exist must be refused");
      for (int layer = 0; layer < LAYERS; ++layer) {
        // rows of the step
        hk.assign(size_t(np) * CHUNK * kv_row, 0), hv = hk, hq.assign(size_t(np) * CHUNK * q_row, 0);
        for (int i = 0; i < np; ++i)
          for (int t = 0; t < plan.prefill[i].n; ++t) {
            const BatchWork& w = plan.prefill[i];
            Row(layer, w.id, w.pos + t, 0, int(kv_row), &hk[(size_t(i) * CHUNK + t) * kv_row], nullptr);
            Row(layer, w.id, w.pos + t, 1, int(kv_row), &hv[(size_t(i) * CHUNK + t) * kv_row], nullptr);
            Row(layer, w.id, w.pos + t, 2, int(q_row), &hq[(size_t(i) * CHUNK + t) * q_row], nullptr);
          }
        if (np > 0) {
          CheckHip(hipMemcpy(pk.get(), hk.data(), hk.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(pv.get(), hv.data(), hv.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(pq.get(), hq.data(), hq.size() * 2, hipMemcpyHostToDevice), "h2d");
        }
        std::vector<uint16_t> k1(size_t(nd) * kv_row), v1(k1.size()), q1(size_t(nd) * q_row);
        for (int i = 0; i < nd; ++i) {
          const BatchWork& w = plan.decode[i];
          Row(layer, w.id, w.pos, 0, int(kv_row), &k1[size_t(i) * kv_row], nullptr);
          Row(layer, w.id, w.pos, 1, int(kv_row), &v1[size_t(i) * kv_row], nullptr);
          Row(layer, w.id, w.pos, 2, int(q_row), &q1[size_t(i) * q_row], nullptr);
        }
        if (nd > 0) {
          CheckHip(hipMemcpy(dk.get(), k1.data(), k1.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(dv.get(), v1.data(), v1.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(dq.get(), q1.data(), q1.size() * 2, hipMemcpyHostToDevice), "h2d");
        }
        b.RunLayer(layer, pk.get(), pv.get(), pq.get(), pout.get(), YAHKV_F32, dk.get(), dv.get(), dq.get(), YAHKV_BF16,
                   static_cast<float*>(dout.get()), YAHKV_BF16, scale);
        CheckHip(hipDeviceSynchronize(), "sync");
        // the oracle, request by request
        std::vector<float> got_p(size_t(np) * CHUNK * q_row), got_d(size_t(nd) * q_row);
        if (np > 0) CheckHip(hipMemcpy(got_p.data(), pout.get(), got_p.size() * 4, hipMemcpyDeviceToHost), "d2h");
        if (nd > 0) CheckHip(hipMemcpy(got_d.data(), dout.get(), got_d.size() * 4, hipMemcpyDeviceToHost), "d2h");
        for (int i = 0; i < np + nd; ++i) {
          const bool pre = i < np;
          const BatchWork& w = pre ? plan.prefill[i] : plan.decode[i - np];
          Mirror& m = mirror.at(w.id)[size_t(layer)];
          std::vector<uint16_t> bits(std::max(kv_row, q_row));
          std::vector<float> kf(size_t(w.n) * kv_row), vf(kf.size()), qf(size_t(w.n) * q_row), want(qf.size());
          for (int t = 0; t < w.n; ++t) {
            Row(layer, w.id, w.pos + t, 0, int(kv_row), bits.data(), &kf[size_t(t) * kv_row]);
            Row(layer, w.id, w.pos + t, 1, int(kv_row), bits.data(), &vf[size_t(t) * kv_row]);
            Row(layer, w.id, w.pos + t, 2, int(q_row), bits.data(), &qf[size_t(t) * q_row]);
          }
          const orc_pools op = m.pools();
          const int32_t pos = w.pos, len = w.pos + w.n;
          orc_append(&m.og, &op, m.table.data(), T / PT, &pos, nullptr, 1, w.n, kf.data(), vf.data());
          if (pre)
            orc_prefill_attend(&m.og, &op, m.table.data(), T / PT, &pos, 1, w.n, qf.data(), scale, nullptr, want.data());
          else
            orc_decode_attend(&m.og, &op, m.table.data(), T / PT, &len, 1, qf.data(), scale, nullptr, want.data());
          const float* got = pre ? &got_p[size_t(i) * CHUNK * q_row] : &got_d[size_t(i - np) * q_row];
          worst = std::max(worst, RelErr(got, want.data(), want.size()));
          m.done = len;
          if (layer == 0) outputs[w.id] += w.n;
        }
        Expect(worst < 2e-3, "attention differs from the oracle");
      }
      b.Commit();
      // requests that ended: their blocks, gathered through the batcher's pages, against the oracle's
      for (int layer = 0; layer < LAYERS; ++layer)
        for (const auto& list : {plan.prefill, plan.decode})
          for (const BatchWork& w : list) {
            const yahkv_pools dp = b.pools(layer);
            const Spec& s = spec[w.id];
            if (w.pos + w.n < s.prompt + s.max_new) continue;
            Mirror& m = mirror.at(w.id)[size_t(layer)];
            const int len = b.length(w.id);
            Expect(len == s.prompt + s.max_new && len == m.done, "a request ends at its full length");
            Expect(outputs[w.id] == len, "one attention row per position");
            const size_t bytes = size_t(len) * H * (D / 32) * 34;
            std::vector<uint8_t> gk(bytes), gv(bytes), wk(bytes), wv(bytes);
            DeviceBuffer bk(bytes), bv(bytes), row(sizeof(int32_t) * b.pages(w.id).size());
            CheckHip(hipMemcpy(row.get(), b.pages(w.id).data(), row.size(), hipMemcpyHostToDevice), "h2d");
            Check(yahkv_gather_blocks(&g, &dp, static_cast<const int32_t*>(row.get()), len, bk.get(), bv.get(), nullptr), "gather");
            CheckHip(hipMemcpy(gk.data(), bk.get(), bytes, hipMemcpyDeviceToHost), "d2h");
            CheckHip(hipMemcpy(gv.data(), bv.get(), bytes, hipMemcpyDeviceToHost), "d2h");
            const orc_pools op = m.pools();
            orc_gather_blocks(&m.og, &op, m.table.data(), len, wk.data(), wv.data());
            Expect(gk == wk && gv == wv, "a finished request's blocks differ from the oracle");
          }
      for (int64_t id : b.TakeFinished()) mirror.erase(id);
    }
    const BatchStats& st = b.stats();
    Expect(mirror.empty() && st.finished == n_req, "every request ends");
    Expect(b.free_pages() == n_pages, "every page is free again");
    Expect(st.preempted > 0, "the pool was meant to run out at least once");
    Expect(st.peak_running >= 3, "requests were meant to run side by side");
    Expect(st.admitted == n_req + st.preempted, "every request put back is admitted again");
    // stopping early: one queued and one running request
    b.Submit(1, 40, 10), b.Submit(2, 20, 10), b.Submit(3, 150, 40), b.Submit(4, 150, 40), b.Submit(5, 150, 40);
    (void)b.Schedule();
    ExpectThrow([&] { b.Stop(1); }, "Stop between Schedule and Commit must throw");
    b.RunLayer(0, pk.get(), pv.get(), pq.get(), pout.get(), YAHKV_F32, dk.get(), dv.get(), dq.get(), YAHKV_BF16,
               static_cast<float*>(dout.get()), YAHKV_BF16, scale);
    b.Commit();
    Expect(b.running() >= 2 && b.queued() >= 1, "some running, some waiting");
    b.Stop(1), b.Stop(5), b.Stop(77);
    const std::vector<int64_t> gone = b.TakeFinished();
    Expect(gone.size() == 2, "two requests stopped");
    b.Stop(2), b.Stop(3), b.Stop(4);
    (void)b.TakeFinished();
    Expect(b.idle() && b.free_pages() == n_pages, "stopped requests give their pages back");
    std::printf("kv_batcher_test: ok (%lld steps, %lld prompt + %lld decode tokens, %lld put back, peak %d running / %d pages, "
                "max relative error %.2e)\n", (long long)st.steps, (long long)st.prefill_tokens, (long long)st.decode_tokens,
                (long long)st.preempted, st.peak_running, st.peak_pages, worst);
    return 0;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "kv_batcher_test: FAILED: %s\n", e.what());
    return 1;
  }
}
}  // namespace

// Every object of the test is gone when RunTest returns. The process then leaves without running the exit handlers:
// the HIP runtime's own teardown has crashed now and then after a test that had passed.
int main() {
  const int rc = RunTest();
  std::fflush(stdout);
  std::fflush(stderr);
  std::_Exit(rc);
}
