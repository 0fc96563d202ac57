// GPU test of the C++ host classes for the reference's own KV formats (csrc/kv8_cache.hpp; kv8a16, then kv4a16) against
// the CPU oracle of those formats (oracle/kv8_oracle.c): two prefill chunks of two sequences (the second chunk starts inside a 16-key tile), then
// decode steps that close tiles and cross a page, a third sequence that starts with decode steps; buffers bit-exact,
// attention within 2e-3 of the float64 closed form over the oracle's dequantized model; and the host checks that throw
// where the reference's LoomDecoder throws (engine/model/loom_decoder.hpp:186-203, 229-235).
#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <string>
#include <vector>

#include "kv8_cache.hpp"
#include "kv8_oracle.h"
#include "yahkv_oracle.h"

using namespace yahkv_host;

namespace {

struct Fail : std::runtime_error {
  using std::runtime_error::runtime_error;
};
void Stage(const char* what) { std::fprintf(stderr, "kv8_cache_test: %s\n", what); }
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

constexpr int H = 2, NQ = 12, D = 256, W = H * D, P = 12;

// softmax(q K^T / 16) V in double over the first n tokens of the dense model; q, out [NQ][D]
void Closed(const std::vector<float>& Kd, const std::vector<float>& Vd, int n, const float* q, double* out) {
  for (int hq = 0; hq < NQ; ++hq) {
    const int h = hq / (NQ / H);
    std::vector<double> sc(static_cast<size_t>(n));
    double mx = -1e300, sum = 0;
    for (int t = 0; t < n; ++t) {
      double d = 0;
      for (int i = 0; i < D; ++i) d += double(Kd[size_t(t) * W + h * D + i]) * q[hq * D + i];
      sc[size_t(t)] = d / 16.0, mx = std::max(mx, sc[size_t(t)]);
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

struct HostPools {
  std::vector<uint32_t> kq, ks, vq, vs;
  std::vector<float> km;
  std::vector<uint16_t> vo;
  HostPools(int kb, int vb)
      : kq(size_t(P) * 256 * W / (kb == 4 ? 8 : 4)), ks(size_t(P) * 256 * W / (kb == 4 ? 32 : 128)),
        vq(size_t(H) * P * 16 * 256 * (vb == 4 ? 2 : 4)), vs(size_t(H) * P * 16 * 256),
        km(size_t(P) * W), vo(size_t(P) * W * 16) {}
  orc_kv8_pools view() { return orc_kv8_pools{kq.data(), ks.data(), km.data(), vq.data(), vs.data(), vo.data()}; }
};

int RunTest(int kb, int vb) {
  try {
    Stage(kb == 8 ? "kv8a16" : "kv4a16");
    const yahkv_geometry g{kb == 8 ? YAHKV_KV8A16 : YAHKV_KV4A16, NQ, H, D, 256, P};
    const orc_kv8_geometry og{NQ, H, P, kb, vb};
    const int B = 2, T = 600, chunk0 = 100, chunk1 = 150, steps = 30;
    std::mt19937 rng(11);
    std::normal_distribution<float> nd;
    auto randn = [&](size_t n, float shift) {
      std::vector<float> v(n);
      for (auto& x : v) x = orc_bf16_to_f32(orc_f32_to_bf16(nd(rng) + shift));
      return v;
    };
    auto to_dev_bf16 = [&](const std::vector<float>& f) {
      std::vector<uint16_t> b(f.size());
      for (size_t i = 0; i < f.size(); ++i) b[i] = orc_f32_to_bf16(f[i]);
      DeviceBuffer d(b.size() * 2);
      CheckHip(hipMemcpy(d.get(), b.data(), b.size() * 2, hipMemcpyHostToDevice), "h2d");
      return d;
    };
    ExpectThrow([&] { Kv8Decoder bad(yahkv_geometry{YAHKV_Q8_0, NQ, H, D, 64, P}, 3, T); }, "a q8_0 geometry is not a kv8a16 one");
    Kv8Decoder dec(g, 3, T);
    ExpectThrow([&] { dec.Step(B, nullptr, nullptr, YAHKV_BF16, nullptr, YAHKV_BF16, 1.0f, nullptr, nullptr); },
                "Step before Bind must throw");
    Kv8DecoderState st = dec.OwnState(/*shuffle_seed=*/5);
    {
      Kv8DecoderState small = st;
      small.vopen.length -= 1;
      ExpectThrow([&] { dec.Bind(small); }, "Bind must reject an open-tile buffer smaller than the geometry");
      small = st, small.km.ptr = nullptr;
      ExpectThrow([&] { dec.Bind(small); }, "Bind must reject a missing buffer");
    }
    dec.Bind(st);
    Expect(dec.KqBytes() == size_t(P) * 256 * W / (kb == 4 ? 2 : 1) && dec.VsBytes() == size_t(P) * 16 * W * 4, "pool byte formulas");
    for (const BufferRef* r : {&st.kq, &st.ks, &st.vq, &st.vs, &st.vopen})  // poison: what is not written stays
      CheckHip(hipMemset(r->ptr, 0x5A, r->length), "poison");
    HostPools hp(kb, vb);
    std::memset(hp.kq.data(), 0x5A, hp.kq.size() * 4), std::memset(hp.ks.data(), 0x5A, hp.ks.size() * 4);
    std::memset(hp.vq.data(), 0x5A, hp.vq.size() * 4), std::memset(hp.vs.data(), 0x5A, hp.vs.size() * 4);
    std::memset(hp.vo.data(), 0x5A, hp.vo.size() * 2);
    const orc_kv8_pools op = hp.view();
    const int stride = dec.page_table_stride();
    std::vector<int32_t> table(size_t(3) * stride, 0);
    auto refresh_table = [&] {
      for (int s = 0; s < 3; ++s)
        for (size_t p = 0; p < dec.pages(s).size(); ++p) table[size_t(s) * stride + p] = dec.pages(s)[p];
    };
    auto pools_equal = [&](const char* what) {
      CheckHip(hipDeviceSynchronize(), "sync");
      struct Pair { const BufferRef* dev; const void* host; size_t bytes; };
      const Pair pairs[6] = {{&st.kq, hp.kq.data(), hp.kq.size() * 4}, {&st.ks, hp.ks.data(), hp.ks.size() * 4},
                             {&st.vq, hp.vq.data(), hp.vq.size() * 4}, {&st.vs, hp.vs.data(), hp.vs.size() * 4},
                             {&st.vopen, hp.vo.data(), hp.vo.size() * 2}, {&st.km, hp.km.data(), hp.km.size() * 4}};
      for (int i = 0; i < 6; ++i) {
        std::vector<uint8_t> got(pairs[i].bytes);
        CheckHip(hipMemcpy(got.data(), pairs[i].dev->ptr, got.size(), hipMemcpyDeviceToHost), "d2h");
        if (i == 5) {  // the means: only the first pages of live sequences are defined
          for (int s = 0; s < 3; ++s)
            if (!dec.pages(s).empty() &&
                std::memcmp(got.data() + size_t(dec.pages(s)[0]) * W * 4, hp.km.data() + size_t(dec.pages(s)[0]) * W, W * 4) != 0)
              throw Fail((std::string(what) + ": channel means differ from the oracle").c_str());
        } else if (std::memcmp(got.data(), pairs[i].host, got.size()) != 0) {
          throw Fail((std::string(what) + ": buffer " + std::to_string(i) + " differs from the oracle").c_str());
        }
      }
    };
    const float scale = 0.0625f;
    Kv8Prefill pre(dec);
    std::vector<int32_t> prefix(B, 0);
    double worst_prefill = 0, worst_decode = 0, worst_twin = 0;
    for (int round = 0; round < 2; ++round) {
      Stage(round == 0 ? "first chunk (channel means, chunk append, attention)" : "second chunk (starts inside a tile)");
      const int chunk = round == 0 ? chunk0 : chunk1;
      const std::vector<float> kf = randn(size_t(B) * chunk * W, 0.6f), vf = randn(size_t(B) * chunk * W, 0.0f);
      const std::vector<float> qf = randn(size_t(B) * chunk * NQ * D, 0.0f);
      DeviceBuffer dk = to_dev_bf16(kf), dv = to_dev_bf16(vf), dq = to_dev_bf16(qf), dout(qf.size() * 4);
      pre.RunChunk(B, chunk, dk.get(), dv.get(), YAHKV_BF16, dq.get(), scale, nullptr, dout.get(), YAHKV_F32);
      refresh_table();
      if (round == 0)
        for (int s = 0; s < B; ++s)
          orc_kv8_kmean(kf.data() + size_t(s) * chunk * W, chunk, W, hp.km.data() + size_t(table[size_t(s) * stride]) * W);
      orc_kv8_append(&og, &op, table.data(), stride, prefix.data(), nullptr, B, chunk, kf.data(), vf.data());
      pools_equal(round == 0 ? "after the first chunk" : "after the second chunk");
      std::vector<float> got(qf.size());
      CheckHip(hipMemcpy(got.data(), dout.get(), got.size() * 4, hipMemcpyDeviceToHost), "d2h");
      for (int s = 0; s < B; ++s) {
        const int n = prefix[size_t(s)] + chunk;
        std::vector<float> Kd(size_t(n) * W), Vd(size_t(n) * W);
        orc_kv8_dense_f16(&og, &op, table.data() + size_t(s) * stride, n, Kd.data(), Vd.data());
        for (int t : {0, 17, chunk - 1}) {
          std::vector<double> want(size_t(NQ) * D);
          const size_t qo = (size_t(s) * chunk + t) * NQ * D;
          Closed(Kd, Vd, prefix[size_t(s)] + t + 1, Rotated(qf.data() + qo, kb, true).data(), want.data());
          worst_prefill = std::max(worst_prefill, RelErr(got.data() + qo, want.data(), want.size()));
        }
        prefix[size_t(s)] = n;
      }
    }
    Expect(worst_prefill < 2e-3, "prefill attention differs from the closed form");
    Expect(dec.length(0) == chunk0 + chunk1 && dec.pages(0).size() == 1, "lengths and pages after the chunks");

    Stage("decode steps (tiles close at 255 and 271, a new page at 256; a third sequence starts from nothing)");
    ExpectThrow([&] { dec.ResumeAt(0, 243); }, "ResumeAt inside a tile the open tile does not cover must throw");
    dec.ResumeAt(0, chunk0 + chunk1);  // where the prefill left the open tile: allowed
    for (int i = 0; i < steps; ++i) {
      const int n_seqs = 3;
      const std::vector<float> k1 = randn(size_t(n_seqs) * W, 0.6f), v1 = randn(size_t(n_seqs) * W, 0.0f);
      const std::vector<float> q1 = randn(size_t(n_seqs) * NQ * D, 0.0f);
      DeviceBuffer dk = to_dev_bf16(k1), dv = to_dev_bf16(v1), dq = to_dev_bf16(q1), dout(q1.size() * 4);
      std::vector<int32_t> pos(n_seqs);
      for (int s = 0; s < n_seqs; ++s) pos[size_t(s)] = dec.length(s);
      dec.Step(n_seqs, dk.get(), dv.get(), YAHKV_BF16, dq.get(), YAHKV_BF16, scale, nullptr, static_cast<float*>(dout.get()));
      CheckHip(hipDeviceSynchronize(), "sync");
      refresh_table();
      if (i == 0) std::memset(hp.km.data() + size_t(table[size_t(2) * stride]) * W, 0, W * 4);  // a fresh sequence: means zero
      orc_kv8_append(&og, &op, table.data(), stride, pos.data(), nullptr, n_seqs, 1, k1.data(), v1.data());
      std::vector<float> got(q1.size());
      CheckHip(hipMemcpy(got.data(), dout.get(), got.size() * 4, hipMemcpyDeviceToHost), "d2h");
      for (int s = 0; s < n_seqs; ++s) {
        const int n = pos[size_t(s)] + 1;
        std::vector<float> Kd(size_t(n) * W), Vd(size_t(n) * W);
        orc_kv8_dense(&og, &op, table.data() + size_t(s) * stride, n, Kd.data(), Vd.data());
        std::vector<double> want(size_t(NQ) * D);
        Closed(Kd, Vd, n, Rotated(q1.data() + size_t(s) * NQ * D, kb, false).data(), want.data());
        worst_decode = std::max(worst_decode, RelErr(got.data() + size_t(s) * NQ * D, want.data(), want.size()));
      }
    }
    pools_equal("after the decode steps");
    Expect(worst_decode < 2e-3, "decode attention differs from the closed form");
    Expect(dec.length(0) == chunk0 + chunk1 + steps && dec.pages(0).size() == 2 && dec.length(2) == steps, "lengths after the steps");
    Stage("fork and slots (sequence 1 becomes a copy of sequence 0, then is loaded from its slot)");
    {
      auto read_file = [](const std::string& path) {
        std::vector<uint8_t> b;
        FILE* f = std::fopen(path.c_str(), "rb");
        if (f == nullptr) throw Fail("a slot file is missing");
        uint8_t buf[1 << 16];
        for (size_t n; (n = std::fread(buf, 1, sizeof buf, f)) > 0;) b.insert(b.end(), buf, buf + n);
        std::fclose(f);
        return b;
      };
      // both sequences take the same rows: the outputs agree up to where the cut places the sequences' tiles (each
      // part rounds its weights to f16 against its own running maximum), and what the steps write is the same byte
      // for byte
      auto twin_steps = [&](int n, const char* what) {
        for (int i = 0; i < n; ++i) {
          std::vector<float> k1 = randn(W, 0.6f), v1 = randn(W, 0.0f), q1 = randn(size_t(NQ) * D, 0.0f);
          k1.insert(k1.end(), k1.begin(), k1.begin() + W), v1.insert(v1.end(), v1.begin(), v1.begin() + W);
          q1.insert(q1.end(), q1.begin(), q1.begin() + size_t(NQ) * D);
          DeviceBuffer dk = to_dev_bf16(k1), dv = to_dev_bf16(v1), dq = to_dev_bf16(q1), dout(q1.size() * 4);
          dec.Step(2, dk.get(), dv.get(), YAHKV_BF16, dq.get(), YAHKV_BF16, scale, nullptr, static_cast<float*>(dout.get()));
          std::vector<float> got(q1.size());
          CheckHip(hipMemcpy(got.data(), dout.get(), got.size() * 4, hipMemcpyDeviceToHost), "d2h");
          double d = 0, m = 0;
          for (size_t j = 0; j < size_t(NQ) * D; ++j)
            d = std::max(d, double(std::fabs(got[j] - got[size_t(NQ) * D + j]))), m = std::max(m, double(std::fabs(got[j])));
          worst_twin = std::max(worst_twin, d / m);
          if (!(d <= 1e-3 * m)) throw Fail((std::string(what) + ": the copy attends differently").c_str());
        }
      };
      const std::string a = "/tmp/yahkv_kv8_cache_test_a.slot", b = "/tmp/yahkv_kv8_cache_test_b.slot";
      auto slots_equal = [&](const char* what) {
        dec.SaveSlot(0, a), dec.SaveSlot(1, b);
        const std::vector<uint8_t> fa = read_file(a), fb = read_file(b);
        if (fa.size() != yahkv_kv8_slot_bytes(&g, int32_t(dec.pages(0).size())) || fa != fb)
          throw Fail((std::string(what) + ": the two sequences' slots differ").c_str());
      };
      ExpectThrow([&] { dec.Fork(0, 1); }, "a fork into a sequence that holds pages must throw");
      dec.Release(1);
      const int32_t free_before = dec.free_pages(), len0 = dec.length(0);
      dec.Fork(0, 1);  // 280 tokens: the first page shared, the second copied with its open tile
      Expect(dec.length(1) == len0 && dec.pages(1).size() == 2 && dec.pages(1)[0] == dec.pages(0)[0] &&
                 dec.pages(1)[1] != dec.pages(0)[1] && dec.free_pages() == free_before - 1, "pages after the fork");
      twin_steps(10, "after the fork");  // to 290: two tiles close
      slots_equal("after the fork");
      dec.Release(1);
      Expect(dec.free_pages() == free_before, "a released fork gives back its own page only");
      ExpectThrow([&] { dec.LoadSlot(0, a); }, "a slot loads into an empty sequence only");
      Expect(dec.LoadSlot(1, a) == len0 + 10 && dec.length(1) == len0 + 10 && dec.pages(1).size() == 2 &&
                 dec.pages(1)[0] != dec.pages(0)[0], "a loaded slot's length and pages");
      twin_steps(250, "after the load");  // past the next page boundary (512)
      slots_equal("after the load");
      Expect(dec.pages(1).size() == 3, "pages after the steps");
      {
        const yahkv_geometry other{kb == 8 ? YAHKV_KV4A16 : YAHKV_KV8A16, NQ, H, D, 256, P};
        Kv8Decoder wrong(other, 1, T);
        wrong.Bind(wrong.OwnState());
        ExpectThrow([&] { wrong.LoadSlot(0, a); }, "a slot of another format must be refused");
        std::vector<uint8_t> cut = read_file(a);
        cut.resize(cut.size() - 1);
        FILE* f = std::fopen(b.c_str(), "wb");
        std::fwrite(cut.data(), 1, cut.size(), f), std::fclose(f);
        dec.Release(1);
        ExpectThrow([&] { dec.LoadSlot(1, b); }, "a truncated slot must be refused");
        Expect(dec.pages(1).empty(), "a refused slot leaves the sequence empty");
      }
      std::remove(a.c_str()), std::remove(b.c_str());
      dec.ResumeAt(1, 0);
    }
    ExpectThrow([&] { dec.ResumeAt(1, 100); dec.Step(2, nullptr, nullptr, YAHKV_BF16, nullptr, YAHKV_BF16, 1.0f, nullptr, nullptr); },
                "a step inside a tile the open tile does not cover must throw");
    dec.Release(0), dec.Release(1), dec.Release(2);
    Expect(dec.free_pages() == P, "every page back in the pool");
    std::printf("kv8_cache_test: ok, kv%da16 (prefill %.2e, decode %.2e, a copy against its source %.2e)\n", kb,
                worst_prefill, worst_decode, worst_twin);
    return 0;
  } catch (const std::exception& e) {
    std::printf("kv8_cache_test: FAILED: %s\n", e.what());
    return 1;
  }
}
}  // namespace

int main() {
  if (const int rc = RunTest(8, 8)) return rc;
  return RunTest(4, 4);
}
