// GPU test of the C++ host classes (csrc/kv_cache.hpp) against the CPU oracle: a chunked prefill of three sequences,
// then decode steps, with pages from the allocator; pools bit-exact, attention within 2e-3; and the host checks that
// throw where the reference's LoomDecoder throws (engine/model/loom_decoder.hpp:186-203,229-235).
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "kv_cache.hpp"
#include "yahkv_oracle.h"

using namespace yahkv_host;

namespace {

uint16_t Bf16(float f) { return orc_f32_to_bf16(f); }
float Widen(uint16_t h) { return orc_bf16_to_f32(h); }

struct Fail : std::runtime_error {
  using std::runtime_error::runtime_error;
};
// stderr is unbuffered: if the program dies, the last stage it names is where
void Stage(const char* what) { std::fprintf(stderr, "kv_cache_test: %s\n", what); }
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
double RelErr(const std::vector<float>& got, const std::vector<float>& want) {
  double d = 0, m = 0;
  for (size_t i = 0; i < got.size(); ++i) d = std::max(d, std::fabs(double(got[i]) - want[i])), m = std::max(m, std::fabs(double(want[i])));
  return d / m;
}

}  // namespace

namespace {
int RunTest() {
  try {
    const yahkv_geometry g{YAHKV_Q8_0, 8, 2, 128, 16, 40};
    const orc_geometry og{8, 8, 2, 128, 16, 40};
    const int B = 3, T = 200, chunk = 37, steps = 5, H = 2, D = 128, NQ = 8;
    std::mt19937 rng(7);
    std::normal_distribution<float> nd;
    auto randn_bf16 = [&](size_t n, std::vector<uint16_t>* bits, std::vector<float>* f) {
      bits->resize(n), f->resize(n);
      for (size_t i = 0; i < n; ++i) (*bits)[i] = Bf16(nd(rng)), (*f)[i] = Widen((*bits)[i]);
    };

    KvDecoder dec(g, B, T);
    ExpectThrow([&] { dec.Step(B, nullptr, nullptr, YAHKV_BF16, nullptr, YAHKV_BF16, 1.0f, nullptr, nullptr); },
                "Step before Bind must throw");
    KvDecoderState st = dec.OwnState(/*shuffle_seed=*/99);
    {
      KvDecoderState small = st;
      small.kq.length -= 1;
      ExpectThrow([&] { dec.Bind(small); }, "Bind must reject a pool smaller than the geometry");
      small = st, small.ptab.length = 4;
      ExpectThrow([&] { dec.Bind(small); }, "Bind must reject a short page table");
    }
    dec.Bind(st);
    Expect(dec.KqBytes() == size_t(40) * 2 * 128 * 16 && dec.KsBytes() == size_t(40) * 2 * 16 * 4 * 2, "pool byte formulas");
    Expect(dec.free_pages() == 40, "fresh pool");

    // ---- prefill chunk
    Stage("prefill chunk");
    std::vector<uint16_t> kb, vb, qb;
    std::vector<float> kf, vf, qf;
    randn_bf16(size_t(B) * chunk * H * D, &kb, &kf);
    randn_bf16(size_t(B) * chunk * H * D, &vb, &vf);
    randn_bf16(size_t(B) * chunk * NQ * D, &qb, &qf);
    DeviceBuffer dk(kb.size() * 2), dv(vb.size() * 2), dq(qb.size() * 2), dout(qb.size() * 4);
    CheckHip(hipMemcpy(dk.get(), kb.data(), kb.size() * 2, hipMemcpyHostToDevice), "h2d");
    CheckHip(hipMemcpy(dv.get(), vb.data(), vb.size() * 2, hipMemcpyHostToDevice), "h2d");
    CheckHip(hipMemcpy(dq.get(), qb.data(), qb.size() * 2, hipMemcpyHostToDevice), "h2d");
    KvPrefill pre(dec);
    const float scale = 1.0f / std::sqrt(float(D));
    pre.RunChunk(B, chunk, dk.get(), dv.get(), YAHKV_BF16, dq.get(), scale, nullptr, dout.get(), YAHKV_F32);
    CheckHip(hipDeviceSynchronize(), "sync");
    Expect(dec.length(0) == chunk && dec.pages(1).size() == 3 && dec.free_pages() == 40 - 9, "pages after the chunk");

    // oracle mirror with the decoder's own page tables
    const int stride = dec.page_table_stride();
    std::vector<int32_t> table(size_t(B) * stride, 0), zero(B, 0), pre_len(B, 0);
    auto refresh_table = [&] {
      for (int s = 0; s < B; ++s)
        for (size_t p = 0; p < dec.pages(s).size(); ++p) table[size_t(s) * stride + p] = dec.pages(s)[p];
    };
    refresh_table();
    std::vector<uint8_t> hkq(orc_kq_bytes(&og), 0), hvq(orc_vq_bytes(&og), 0);
    std::vector<uint16_t> hks(orc_ks_bytes(&og) / 2, 0), hvs(orc_vs_bytes(&og) / 2, 0);
    const orc_pools op{hkq.data(), hks.data(), hvq.data(), hvs.data()};
    orc_append(&og, &op, table.data(), stride, zero.data(), nullptr, B, chunk, kf.data(), vf.data());
    std::vector<float> want(qf.size()), got(qf.size());
    orc_prefill_attend(&og, &op, table.data(), stride, pre_len.data(), B, chunk, qf.data(), scale, nullptr, want.data());
    CheckHip(hipMemcpy(got.data(), dout.get(), got.size() * 4, hipMemcpyDeviceToHost), "d2h");
    const double e1 = RelErr(got, want);
    Expect(e1 < 2e-3, "prefill attention differs from the oracle");

    // ---- decode steps: all of them queued back to back, no host wait in between (the positions of a step travel
    // through staging memory that the next step must not overwrite before its copy has run), then every step's output
    // against the oracle
    Stage("decode steps");
    double e2 = 0;
    {
      const size_t kv_n = size_t(B) * H * D, q_n = size_t(B) * NQ * D;
      std::vector<std::vector<float>> k1f(steps), v1f(steps), q1f(steps);
      DeviceBuffer sk(kv_n * 2 * steps), sv(kv_n * 2 * steps), sq(q_n * 2 * steps), sout(q_n * 4 * steps);
      for (int i = 0; i < steps; ++i) {
        std::vector<uint16_t> k1, v1, q1;
        randn_bf16(kv_n, &k1, &k1f[i]);
        randn_bf16(kv_n, &v1, &v1f[i]);
        randn_bf16(q_n, &q1, &q1f[i]);
        CheckHip(hipMemcpy(static_cast<char*>(sk.get()) + kv_n * 2 * i, k1.data(), kv_n * 2, hipMemcpyHostToDevice), "h2d");
        CheckHip(hipMemcpy(static_cast<char*>(sv.get()) + kv_n * 2 * i, v1.data(), kv_n * 2, hipMemcpyHostToDevice), "h2d");
        CheckHip(hipMemcpy(static_cast<char*>(sq.get()) + q_n * 2 * i, q1.data(), q_n * 2, hipMemcpyHostToDevice), "h2d");
      }
      // the set-up call a server makes once: the XCDs' shares for this batch (a batch too small for whole groups of
      // chunks keeps equal shares); the steps below must come out the same either way
      dec.Calibrate(B, sq.get(), YAHKV_BF16, 2);
      for (int j = 0; j < 8; ++j)
        if (dec.options().xcd_weight[j] < 0) throw std::runtime_error("calibration left a negative weight");
      std::vector<std::vector<int32_t>> pos(steps, std::vector<int32_t>(B)), len(steps, std::vector<int32_t>(B));
      for (int i = 0; i < steps; ++i) {
        for (int s = 0; s < B; ++s) pos[i][s] = dec.length(s), len[i][s] = pos[i][s] + 1;
        dec.Step(B, static_cast<char*>(sk.get()) + kv_n * 2 * i, static_cast<char*>(sv.get()) + kv_n * 2 * i, YAHKV_BF16,
                 static_cast<char*>(sq.get()) + q_n * 2 * i, YAHKV_BF16, scale, nullptr,
                 reinterpret_cast<float*>(static_cast<char*>(sout.get()) + q_n * 4 * i));
      }
      CheckHip(hipDeviceSynchronize(), "sync");
      refresh_table();
      for (int i = 0; i < steps; ++i) {
        orc_append(&og, &op, table.data(), stride, pos[i].data(), nullptr, B, 1, k1f[i].data(), v1f[i].data());
        std::vector<float> w(q_n), o(q_n);
        orc_decode_attend(&og, &op, table.data(), stride, len[i].data(), B, q1f[i].data(), scale, nullptr, w.data());
        CheckHip(hipMemcpy(o.data(), static_cast<char*>(sout.get()) + q_n * 4 * i, q_n * 4, hipMemcpyDeviceToHost), "d2h");
        e2 = std::max(e2, RelErr(o, w));
      }
    }
    Expect(e2 < 2e-3, "decode attention differs from the oracle");
    // pool contents bit-exact: every sequence's blocks, gathered through the page table, against the oracle's
    const yahkv_pools dp = yahkv_host::PoolsOf(st);
    for (int s = 0; s < B; ++s) {
      const size_t bytes = size_t(dec.length(s)) * H * (D / 32) * 34;
      std::vector<uint8_t> gk(bytes), gv(bytes), wk(bytes), wv(bytes);
      DeviceBuffer bk(bytes), bv(bytes);
      Check(yahkv_gather_blocks(&g, &dp, static_cast<const int32_t*>(st.ptab.ptr) + size_t(s) * stride, dec.length(s),
                                bk.get(), bv.get(), nullptr), "gather");
      CheckHip(hipMemcpy(gk.data(), bk.get(), bytes, hipMemcpyDeviceToHost), "d2h");
      CheckHip(hipMemcpy(gv.data(), bv.get(), bytes, hipMemcpyDeviceToHost), "d2h");
      orc_gather_blocks(&og, &op, table.data() + size_t(s) * stride, dec.length(s), wk.data(), wv.data());
      Expect(gk == wk && gv == wv, "pool blocks differ from the oracle");
    }

    // ---- host checks
    Stage("host checks");
    Expect(dec.length(2) == chunk + steps, "lengths after the steps");
    ExpectThrow([&] { dec.Reserve(0, T + 1); }, "Reserve past the context must throw");
    const int before = dec.free_pages();
    dec.Release(1);
    Expect(dec.free_pages() == before + 3 && dec.length(1) == 0, "Release returns the pages");
    ExpectThrow([&] { dec.Reserve(1, 16 * (dec.free_pages() + 1)); }, "an exhausted pool must throw");
    dec.ResumeAt(1, 20);
    Expect(dec.length(1) == 20 && dec.pages(1).size() == 2, "ResumeAt reserves the pages below pos");
    KvDecoder tiny(g, 1, 16);
    tiny.Bind(tiny.OwnState());
    tiny.ResumeAt(0, 16);
    ExpectThrow([&] { tiny.Step(1, dk.get(), dv.get(), YAHKV_BF16, dq.get(), YAHKV_BF16, scale, nullptr, static_cast<float*>(dout.get())); },
                "Step past the context must throw");
    // ---- fork (shared prefix pages) and slot files
    Stage("fork and slots");
    {
      auto gathered = [&](KvDecoder& d, int seq) {
        const size_t bytes = size_t(d.length(seq)) * H * (D / 32) * 34;
        std::vector<uint8_t> k(bytes), v(bytes);
        DeviceBuffer bk(bytes), bv(bytes);
        const yahkv_pools pp = yahkv_host::PoolsOf(d.state());
        d.Upload();
        Check(yahkv_gather_blocks(&g, &pp, static_cast<const int32_t*>(d.state().ptab.ptr) + size_t(seq) * d.page_table_stride(),
                                  d.length(seq), bk.get(), bv.get(), nullptr), "gather");
        CheckHip(hipMemcpy(k.data(), bk.get(), bytes, hipMemcpyDeviceToHost), "d2h");
        CheckHip(hipMemcpy(v.data(), bv.get(), bytes, hipMemcpyDeviceToHost), "d2h");
        k.insert(k.end(), v.begin(), v.end());
        return k;
      };
      dec.Release(1);
      const int free0 = dec.free_pages();
      const int len2 = dec.length(2), full = len2 / 16, partial = len2 % 16 != 0;
      dec.Fork(2, 1);
      Expect(dec.length(1) == len2 && dec.free_pages() == free0 - partial, "a fork takes one page at most");
      for (int i = 0; i < full; ++i) Expect(dec.pages(1)[size_t(i)] == dec.pages(2)[size_t(i)], "full pages are shared");
      if (partial) Expect(dec.pages(1).back() != dec.pages(2).back(), "the partly filled page is private");
      Expect(gathered(dec, 1) == gathered(dec, 2), "a fork holds the same blocks");
      dec.Release(2);  // the parent goes: the shared pages stay with the child
      Expect(dec.free_pages() == free0 - partial + partial, "the parent's private page comes back");
      const std::vector<uint8_t> child = gathered(dec, 1);
      const std::string path = "/tmp/yahkv_kv_cache_test.slot";
      dec.SaveSlot(1, path);
      KvDecoder other(g, 2, T);
      other.Bind(other.OwnState(7));
      Expect(other.LoadSlot(1, path) == len2, "LoadSlot returns the tokens it covers");
      Expect(gathered(other, 1) == child, "a loaded slot holds the same blocks");
      yahkv_geometry g2 = g;
      g2.page_tokens = 32;
      KvDecoder wrong(g2, 1, T);
      wrong.Bind(wrong.OwnState());
      ExpectThrow([&] { wrong.LoadSlot(0, path); }, "a slot of another geometry must be refused");
      std::remove(path.c_str());
    }
    Stage("done");
    std::printf("kv_cache_test: ok (prefill %.2e, decode %.2e max relative error)\n", e1, e2);
    std::fflush(stdout);
    return 0;
  } catch (const std::exception& e) {
    std::fprintf(stderr, "kv_cache_test: FAILED: %s\n", e.what());
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
