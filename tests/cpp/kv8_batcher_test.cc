// GPU test of the continuous-batching driver over pools in the reference's own formats (csrc/kv8_batcher.hpp; kv8a16,
// then kv4a16) against the CPU oracle of those formats (oracle/kv8_oracle.c). Ten requests with prompts of 3 to 520
// tokens and 0 to 40 generated tokens go through five pages, which cannot hold them all: requests wait, take their
// prompts in chunks of 100 (so chunks start inside 16-key tiles and inside pages) next to decoding ones, are put back
// and start again; first chunks and later chunks share a step. Two layers share the page table. Every row is a
// function of (layer, request, position) alone. The oracle follows the batcher's page tables in host pools that start
// from the same fill, so after every step all six buffers of both layers are compared whole, bit for bit (the means
// and open tiles of requests that wait or were put back included); attention rows within 2e-3 of the float64 closed
// form over the oracle's dequantized model.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <random>
#include <string>
#include <vector>

#include "kv8_batcher.hpp"
#include "kv8_oracle.h"
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

constexpr int NQ = 8, H = 2, D = 256, W = H * D, PT = 256, T = 768, CHUNK = 100, LAYERS = 2, P = 5;

// Row `kind` (0 K, 1 V, 2 Q) of (layer, request, position): bf16 normals (K around 0.6) from a generator seeded by the
// triple.
void Row(int layer, int64_t id, int pos, int kind, int n, uint16_t* bits, float* f) {
  std::mt19937 rng(uint32_t(id * 7919 + pos * 31 + kind * 1000003 + layer * 50021 + 17));
  std::normal_distribution<float> nd;
  for (int i = 0; i < n; ++i) {
    const uint16_t b = orc_f32_to_bf16(nd(rng) + (kind == 0 ? 0.6f : 0.0f));
    if (bits != nullptr) bits[i] = b;
    if (f != nullptr) f[i] = orc_bf16_to_f32(b);
  }
}

// softmax(q K^T * scale) V in double over the first n tokens of the dense model; q, out [NQ][D]
void Closed(const std::vector<float>& Kd, const std::vector<float>& Vd, int n, const float* q, double scale, double* out) {
  for (int hq = 0; hq < NQ; ++hq) {
    const int h = hq / (NQ / H);
    std::vector<double> sc(static_cast<size_t>(n));
    double mx = -1e300, sum = 0;
    for (int t = 0; t < n; ++t) {
      double d = 0;
      for (int i = 0; i < D; ++i) d += double(Kd[size_t(t) * W + h * D + i]) * q[hq * D + i];
      sc[size_t(t)] = d * scale, mx = std::max(mx, sc[size_t(t)]);
    }
    for (int t = 0; t < n; ++t) sc[size_t(t)] = std::exp(sc[size_t(t)] - mx), sum += sc[size_t(t)];
    for (int i = 0; i < D; ++i) {
      double a = 0;
      for (int t = 0; t < n; ++t) a += sc[size_t(t)] * Vd[size_t(t) * W + h * D + i];
      out[hq * D + i] = a / sum;
    }
  }
}
// what the attention over 4-bit K scores against: H256 q / 16 per head, the prefill's rounded to f16 (yah_qrot)
std::vector<float> Rotated(const float* q, int kb, bool to_f16) {
  std::vector<float> out(q, q + size_t(NQ) * D);
  if (kb != 4) return out;
  for (int hq = 0; hq < NQ; ++hq) {
    orc_kv4_rotate_q(q + hq * D, out.data() + hq * D);
    if (to_f16)
      for (int i = 0; i < D; ++i) out[size_t(hq) * D + i] = orc_f16_to_f32(orc_f32_to_f16(out[size_t(hq) * D + i]));
  }
  return out;
}
double RelErr(const float* got, const double* want, size_t n) {
  double d = 0, m = 0;
  for (size_t i = 0; i < n; ++i) d = std::max(d, std::fabs(got[i] - want[i])), m = std::max(m, std::fabs(want[i]));
  return d / m;
}

// One layer's pools on the host, in the device's layouts, filled like the device's before the first step.
struct HostPools {
  std::vector<uint32_t> kq, ks, vq, vs;
  std::vector<float> km;
  std::vector<uint16_t> vo;
  HostPools(int kb, int vb)
      : kq(size_t(P) * 256 * W / (kb == 4 ? 8 : 4)), ks(size_t(P) * 256 * W / (kb == 4 ? 32 : 128)),
        vq(size_t(H) * P * 16 * 256 * (vb == 4 ? 2 : 4)), vs(size_t(H) * P * 16 * 256), km(size_t(P) * W),
        vo(size_t(P) * W * 16) {
    for (auto* v : {&kq, &ks, &vq, &vs}) std::memset(v->data(), 0x5A, v->size() * 4);
    std::memset(km.data(), 0x5A, km.size() * 4), std::memset(vo.data(), 0x5A, vo.size() * 2);
  }
  orc_kv8_pools view() { return orc_kv8_pools{kq.data(), ks.data(), km.data(), vq.data(), vs.data(), vo.data()}; }
};

int RunTest(int kb, int vb) {
  try {
    const yahkv_geometry g{kb == 8 ? YAHKV_KV8A16 : YAHKV_KV4A16, NQ, H, D, PT, P};
    const orc_kv8_geometry og{NQ, H, P, kb, vb};
    const int max_running = 4, max_prefill = 2, stride = T / PT;
    ExpectThrow([&] { Kv8Batcher bad(yahkv_geometry{YAHKV_Q8_0, NQ, H, D, 64, P}, 1, 2, T, CHUNK, 1); },
                "a q8_0 geometry is not one of these formats");
    Kv8Batcher b(g, LAYERS, max_running, T, CHUNK, max_prefill, nullptr, /*shuffle_seed=*/5);
    ExpectThrow([&] { b.RunLayer(0, nullptr, nullptr, nullptr, nullptr, YAHKV_F32, nullptr, nullptr, nullptr, YAHKV_BF16, nullptr, YAHKV_BF16, 1.0f); },
                "RunLayer without Schedule must throw");
    std::vector<HostPools> host;
    for (int l = 0; l < LAYERS; ++l) {
      host.emplace_back(kb, vb);
      const yahkv_kv8_pools dp = b.pools(l);
      void* ptr[6] = {dp.kq, dp.ks, dp.km, dp.vq, dp.vs, dp.vopen};
      const size_t len[6] = {dp.kq_bytes, dp.ks_bytes, dp.km_bytes, dp.vq_bytes, dp.vs_bytes, dp.vopen_bytes};
      for (int i = 0; i < 6; ++i) CheckHip(hipMemset(ptr[i], 0x5A, len[i]), "fill");
    }
    auto pools_equal = [&](int layer) {
      const yahkv_kv8_pools dp = b.pools(layer);
      HostPools& hp = host[size_t(layer)];
      const void* dev[6] = {dp.kq, dp.ks, dp.km, dp.vq, dp.vs, dp.vopen};
      const void* want[6] = {hp.kq.data(), hp.ks.data(), hp.km.data(), hp.vq.data(), hp.vs.data(), hp.vo.data()};
      const size_t len[6] = {hp.kq.size() * 4, hp.ks.size() * 4, hp.km.size() * 4, hp.vq.size() * 4, hp.vs.size() * 4, hp.vo.size() * 2};
      const size_t dev_len[6] = {dp.kq_bytes, dp.ks_bytes, dp.km_bytes, dp.vq_bytes, dp.vs_bytes, dp.vopen_bytes};
      static const char* const name[6] = {"kq", "ks", "km", "vq", "vs", "vopen"};
      for (int i = 0; i < 6; ++i) {
        if (len[i] != dev_len[i]) throw Fail((std::string("the size of ") + name[i] + " differs from the oracle's").c_str());
        std::vector<uint8_t> got(len[i]);
        CheckHip(hipMemcpy(got.data(), dev[i], len[i], hipMemcpyDeviceToHost), "d2h");
        if (std::memcmp(got.data(), want[i], len[i]) != 0)
          throw Fail((std::string("buffer ") + name[i] + " of layer " + std::to_string(layer) + " differs from the oracle").c_str());
      }
    };

    std::mt19937 rng(23);
    struct Spec { int prompt, max_new; };
    std::map<int64_t, Spec> spec;
    std::map<int64_t, int> done, outputs;
    const int n_req = 10;
    for (int64_t id = 100; id < 100 + n_req; ++id) {
      Spec s{int(3 + rng() % 518), int(rng() % 41)};
      if (id == 100) s = Spec{500, 30};  // two long ones, three pages each: the second is put back
      if (id == 101) s = Spec{520, 40};
      if (id == 103) s = Spec{300, 20};
      if (id == 102) s = Spec{1, 20};    // a prompt of one token
      if (id == 104) s = Spec{201, 0};   // ends with its prompt, the last chunk one token long
      if (id == 106) s = Spec{250, 30};  // decode steps cross a page boundary
      spec[id] = s;
    }
    const size_t kv_row = size_t(W), q_row = size_t(NQ) * D;
    DeviceBuffer pk(max_prefill * CHUNK * kv_row * 2), pv(max_prefill * CHUNK * kv_row * 2), pq(max_prefill * CHUNK * q_row * 2);
    DeviceBuffer pout(max_prefill * CHUNK * q_row * 4);
    DeviceBuffer dk(max_running * kv_row * 2), dv(max_running * kv_row * 2), dq(max_running * q_row * 2), dout(max_running * q_row * 4);
    const float scale = 0.0625f;
    double worst_prefill = 0, worst_decode = 0;
    int64_t next_submit = 100;
    int steps = 0, mixed_steps = 0;
    auto arrive = [&](int n) {
      for (; n > 0 && next_submit < 100 + n_req; --n, ++next_submit) {
        b.Submit(next_submit, spec[next_submit].prompt, spec[next_submit].max_new);
        done[next_submit] = 0;
      }
    };
    arrive(4);
    while (!b.idle() || next_submit < 100 + n_req) {
      if (steps % 3 == 1) arrive(1);
      Expect(++steps < 3000, "the batcher makes no progress");
      const BatchPlan plan = b.Schedule();
      const int np = int(plan.prefill.size()), nd = int(plan.decode.size());
      Expect(np <= max_prefill && nd <= max_running && b.running() <= max_running, "plan within the limits");
      int firsts = 0;
      for (const auto& list : {plan.prefill, plan.decode})
        for (const BatchWork& w : list) {
          if (w.pos == 0 && done.at(w.id) != 0) done[w.id] = 0, outputs[w.id] = 0;  // put back: starts again
          Expect(w.pos == done.at(w.id), "work continues where the request stands");
          firsts += w.pos == 0;
        }
      mixed_steps += np == 2 && firsts == 1;
      std::vector<int32_t> table(size_t(np + nd) * stride, 0);
      for (int i = 0; i < np + nd; ++i) {
        const BatchWork& w = i < np ? plan.prefill[size_t(i)] : plan.decode[size_t(i - np)];
        std::copy(b.pages(w.id).begin(), b.pages(w.id).end(), table.begin() + size_t(i) * stride);
      }
      for (int layer = 0; layer < LAYERS; ++layer) {
        // the step's rows: bits for the device, the same values in f32 for the oracle (rows past a chunk's n zero)
        std::vector<uint16_t> hk(size_t(np) * CHUNK * kv_row, 0), hv(hk.size(), 0), hq(size_t(np) * CHUNK * q_row, 0);
        std::vector<float> fk(hk.size(), 0.0f), fv(hk.size(), 0.0f), fq(hq.size(), 0.0f);
        for (int i = 0; i < np; ++i)
          for (int t = 0; t < plan.prefill[size_t(i)].n; ++t) {
            const BatchWork& w = plan.prefill[size_t(i)];
            const size_t r = size_t(i) * CHUNK + t;
            Row(layer, w.id, w.pos + t, 0, int(kv_row), &hk[r * kv_row], &fk[r * kv_row]);
            Row(layer, w.id, w.pos + t, 1, int(kv_row), &hv[r * kv_row], &fv[r * kv_row]);
            Row(layer, w.id, w.pos + t, 2, int(q_row), &hq[r * q_row], &fq[r * q_row]);
          }
        std::vector<uint16_t> k1(size_t(nd) * kv_row), v1(k1.size()), q1(size_t(nd) * q_row);
        std::vector<float> fk1(k1.size()), fv1(k1.size()), fq1(q1.size());
        for (int i = 0; i < nd; ++i) {
          const BatchWork& w = plan.decode[size_t(i)];
          Row(layer, w.id, w.pos, 0, int(kv_row), &k1[size_t(i) * kv_row], &fk1[size_t(i) * kv_row]);
          Row(layer, w.id, w.pos, 1, int(kv_row), &v1[size_t(i) * kv_row], &fv1[size_t(i) * kv_row]);
          Row(layer, w.id, w.pos, 2, int(q_row), &q1[size_t(i) * q_row], &fq1[size_t(i) * q_row]);
        }
        if (np > 0) {
          CheckHip(hipMemcpy(pk.get(), hk.data(), hk.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(pv.get(), hv.data(), hv.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(pq.get(), hq.data(), hq.size() * 2, hipMemcpyHostToDevice), "h2d");
        }
        if (nd > 0) {
          CheckHip(hipMemcpy(dk.get(), k1.data(), k1.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(dv.get(), v1.data(), v1.size() * 2, hipMemcpyHostToDevice), "h2d");
          CheckHip(hipMemcpy(dq.get(), q1.data(), q1.size() * 2, hipMemcpyHostToDevice), "h2d");
        }
        b.RunLayer(layer, pk.get(), pv.get(), pq.get(), pout.get(), YAHKV_F32, dk.get(), dv.get(), dq.get(), YAHKV_BF16,
                   static_cast<float*>(dout.get()), YAHKV_BF16, scale);
        CheckHip(hipDeviceSynchronize(), "sync");
        std::vector<float> got_p(size_t(np) * CHUNK * q_row), got_d(size_t(nd) * q_row);
        if (np > 0) CheckHip(hipMemcpy(got_p.data(), pout.get(), got_p.size() * 4, hipMemcpyDeviceToHost), "d2h");
        if (nd > 0) CheckHip(hipMemcpy(got_d.data(), dout.get(), got_d.size() * 4, hipMemcpyDeviceToHost), "d2h");

        // the oracle, request by request, through the batcher's page table
        HostPools& hp = host[size_t(layer)];
        const orc_kv8_pools op = hp.view();
        for (int i = 0; i < np; ++i) {
          const BatchWork& w = plan.prefill[size_t(i)];
          const int32_t* row = table.data() + size_t(i) * stride;
          const float* kf = fk.data() + size_t(i) * CHUNK * kv_row;
          if (w.pos == 0) orc_kv8_kmean(kf, w.n, W, hp.km.data() + size_t(row[0]) * W);
          const int32_t pos = w.pos, n = w.n;
          orc_kv8_append(&og, &op, row, stride, &pos, &n, 1, CHUNK, kf, fv.data() + size_t(i) * CHUNK * kv_row);
          const int len = w.pos + w.n;
          std::vector<float> Kd(size_t(len) * W), Vd(size_t(len) * W);
          orc_kv8_dense_f16(&og, &op, row, len, Kd.data(), Vd.data());
          for (int t : {0, 17, w.n - 1}) {
            if (t >= w.n) continue;
            std::vector<double> want(q_row);
            const size_t qo = (size_t(i) * CHUNK + t) * q_row;
            Closed(Kd, Vd, w.pos + t + 1, Rotated(fq.data() + qo, kb, true).data(), scale, want.data());
            worst_prefill = std::max(worst_prefill, RelErr(got_p.data() + qo, want.data(), want.size()));
          }
          if (layer == 0) outputs[w.id] += w.n;
        }
        for (int i = 0; i < nd; ++i) {
          const BatchWork& w = plan.decode[size_t(i)];
          const int32_t* row = table.data() + size_t(np + i) * stride;
          const int32_t pos = w.pos;
          orc_kv8_append(&og, &op, row, stride, &pos, nullptr, 1, 1, fk1.data() + size_t(i) * kv_row, fv1.data() + size_t(i) * kv_row);
          const int len = w.pos + 1;
          std::vector<float> Kd(size_t(len) * W), Vd(size_t(len) * W);
          orc_kv8_dense(&og, &op, row, len, Kd.data(), Vd.data());
          std::vector<double> want(q_row);
          Closed(Kd, Vd, len, Rotated(fq1.data() + size_t(i) * q_row, kb, false).data(), scale, want.data());
          worst_decode = std::max(worst_decode, RelErr(got_d.data() + size_t(i) * q_row, want.data(), want.size()));
          if (layer == 0) outputs[w.id] += 1;
        }
        pools_equal(layer);  // (first: bytes that differ say more than the attention over them)
        if (!(worst_prefill < 2e-3 && worst_decode < 2e-3))
          throw Fail(("attention differs from the closed form: prefill " + std::to_string(worst_prefill) + ", decode " +
                      std::to_string(worst_decode) + " at layer " + std::to_string(layer))
                         .c_str());
      }
      b.Commit();
      for (const auto& list : {plan.prefill, plan.decode})
        for (const BatchWork& w : list) {
          done[w.id] = w.pos + w.n;
          const Spec& s = spec[w.id];
          if (w.pos + w.n < s.prompt + s.max_new) continue;
          Expect(b.length(w.id) == s.prompt + s.max_new, "a request ends at its full length");
          Expect(outputs[w.id] == s.prompt + s.max_new, "one attention row per position");
        }
      for (int64_t id : b.TakeFinished()) done.erase(id);
    }
    const BatchStats& st = b.stats();
    Expect(done.empty() && st.finished == n_req, "every request ends");
    Expect(b.free_pages() == P, "every page is free again");
    Expect(st.preempted > 0, "the pool was meant to run out at least once");
    Expect(st.peak_running >= 3, "requests were meant to run side by side");
    Expect(mixed_steps > 0, "a first chunk and a later chunk were meant to share a step");
    std::printf("kv8_batcher_test: ok, kv%da16 (%lld steps, %lld prompt + %lld decode tokens, %lld put back, peak %d running / %d "
                "pages, prefill %.2e, decode %.2e)\n", kb, (long long)st.steps, (long long)st.prefill_tokens,
                (long long)st.decode_tokens, (long long)st.preempted, st.peak_running, st.peak_pages, worst_prefill, worst_decode);
    return 0;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "kv8_batcher_test: FAILED (kv%da16): %s\n", kb, e.what());
    return 1;
  }
}
}  // namespace

// Every object of the test is gone when RunTest returns. The process then leaves without running the exit handlers:
// the HIP runtime's own teardown has crashed now and then after a test that had passed.
int main() {
  int rc = RunTest(8, 8);
  if (rc == 0) rc = RunTest(4, 4);
  std::fflush(stdout);
  std::fflush(stderr);
  std::_Exit(rc);
}
