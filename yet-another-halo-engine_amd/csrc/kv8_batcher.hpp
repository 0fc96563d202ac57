// Continuous batching (kv_batcher.hpp) over pools in the reference's own formats, kv8a16 / kv4a16 and the mixes: the
// same scheduler and step table, the layers' six buffers under one page table, and the format's own per-chunk order
// (loom_prefill.hpp:3343-3410): channel means from a request's first chunk only, the chunk's K and V quantized with
// the newest tile left open, causal attention over prefix + chunk; per decode token kappend, vappend, part_q, reduce
// (loom_decoder.hpp:253-268). A request's means live with its first page and its open tile with its newest, so
// requests that wait, run side by side or start again after being put back do not touch each other's.
//
// The rule of loom_decoder.hpp:233-235 (steps over quantized V are contiguous from a 16-key boundary unless the open
// tile was seeded) holds by construction: a request's positions are planned in order, a chunk leaves its newest tile
// in the open tile, and a request that is put back starts again from its first token.
//
// Header-only, host code only; one host thread, one stream.
#ifndef YAHKV_KV8_BATCHER_HPP_
#define YAHKV_KV8_BATCHER_HPP_

#include "kv8_cache.hpp"
#include "kv_batcher.hpp"

namespace yahkv_host {

class Kv8Batcher {
 public:
  // g.n_pages pages of 256 tokens per layer; the layers share the page table.
  Kv8Batcher(const yahkv_geometry& g, int32_t n_layers, int32_t max_running, int32_t context, int32_t chunk,
             int32_t max_prefill, hipStream_t stream = nullptr, uint64_t shuffle_seed = 0)
      : g_(g), stream_(stream),
        sched_(g.n_pages, g.page_tokens, max_running, context, chunk, max_prefill, shuffle_seed),
        stage_(g, max_running, max_prefill, context, stream) {
    if (yahkv_kv8_kq_bytes(&g_) == 0) throw KvError("kv8 batcher: not a kv8a16 / kv4a16 geometry (head_dim 256, 256-token pages)");
    if (n_layers <= 0 || chunk < 2) throw KvError("kv8 batcher: bad sizes");  // a chunk of one row is a decode append
    const size_t bytes[6] = {yahkv_kv8_kq_bytes(&g_), yahkv_kv8_ks_bytes(&g_), yahkv_kv8_km_bytes(&g_),
                             yahkv_kv8_vq_bytes(&g_), yahkv_kv8_vs_bytes(&g_), yahkv_kv8_vopen_bytes(&g_)};
    for (int32_t l = 0; l < n_layers; ++l) {
      layers_.emplace_back();
      for (int i = 0; i < 6; ++i) layers_.back().buf[i] = DeviceBuffer(bytes[i]);
    }
    workspace_ = DeviceBuffer(yahkv_kv8_decode_workspace_bytes(&g_, max_running, context, nullptr));
  }
  Kv8Batcher(const Kv8Batcher&) = delete;
  Kv8Batcher& operator=(const Kv8Batcher&) = delete;

  void Submit(int64_t id, int32_t prompt_len, int32_t max_new) { sched_.Submit(id, prompt_len, max_new); }
  void Stop(int64_t id) { sched_.Stop(id); }
  std::vector<int64_t> TakeFinished() { return sched_.TakeFinished(); }

  // Plans the step (BatchScheduler::Schedule), checks the page table it implies and sends it to the device.
  const BatchPlan& Schedule() {
    const BatchPlan& plan = sched_.Schedule();
    if (!plan.empty()) stage_.Upload(sched_, plan);
    return plan;
  }

  // Runs the planned step for one layer on the stream; rows in the plan's order, as KvBatcher::RunLayer's:
  //   prompt chunks: pk, pv [n_prefill][chunk][n_kv][256] of kv_dtype, pq [n_prefill][chunk][n_q][256] bf16,
  //                  pout [n_prefill][chunk][n_q][256] of pout_dtype; rows past a chunk's n are ignored / undefined
  //   decode tokens: dk, dv [n_decode][1][n_kv][256] of kv_dtype, dq [n_decode][n_q][256] of dq_dtype, dout f32
  void RunLayer(int32_t layer, const void* pk, const void* pv, const void* pq, void* pout, int32_t pout_dtype,
                const void* dk, const void* dv, const void* dq, int32_t dq_dtype, float* dout, int32_t kv_dtype,
                float softmax_scale) {
    if (!sched_.planned()) throw KvError("kv8 batcher: RunLayer without Schedule");
    if (layer < 0 || layer >= int32_t(layers_.size())) throw KvError("kv8 batcher: no such layer");
    const BatchPlan& plan = sched_.plan();
    const int32_t np = int32_t(plan.prefill.size()), nd = int32_t(plan.decode.size());
    if (np + nd == 0) return;
    const yahkv_kv8_pools pools = this->pools(layer);
    const int32_t chunk = sched_.chunk(), T = sched_.context(), stride = stage_.stride();
    if (np > 0) {
      if (pk == nullptr || pv == nullptr || pq == nullptr || pout == nullptr) throw KvError("kv8 batcher: prompt rows missing");
      const size_t elt = kv_dtype == YAHKV_F32 ? 4 : 2, row = size_t(chunk) * g_.n_kv_heads * 256 * elt;
      // yah_kmean on a request's first chunk only (loom_prefill.hpp:3343-3345): one call per run of such rows
      for (int32_t i = 0; i < np;) {
        if (plan.prefill[size_t(i)].pos != 0) {
          ++i;
          continue;
        }
        int32_t j = i + 1;
        while (j < np && plan.prefill[size_t(j)].pos == 0) ++j;
        Check(yahkv_kv8_kmean(&g_, &pools, stage_.table() + size_t(i) * stride, stride, stage_.valid() + i, j - i, chunk,
                              static_cast<const char*>(pk) + size_t(i) * row, kv_dtype, stream_), "kv8_kmean");
        i = j;
      }
      Check(yahkv_kv8_append(&g_, &pools, stage_.table(), stride, stage_.prefix(), stage_.valid(), np, chunk, pk, pv,
                             kv_dtype, stream_), "kv8_append");
      const size_t need = yahkv_kv8_prefill_workspace_bytes(&g_, np, stage_.max_prefix(), chunk);
      if (need > images_.size()) {
        CheckHip(hipStreamSynchronize(stream_), "prefill workspace");
        images_ = DeviceBuffer(need);
      }
      Check(yahkv_kv8_prefill_attend(&g_, &pools, stage_.table(), stride, stage_.prefix(), np, stage_.max_prefix(), chunk,
                                     pq, softmax_scale, nullptr, pout, pout_dtype, images_.get(), images_.size(), stream_),
            "kv8_prefill_attend");
    }
    if (nd > 0) {
      if (dk == nullptr || dv == nullptr || dq == nullptr || dout == nullptr) throw KvError("kv8 batcher: decode rows missing");
      Check(yahkv_kv8_decode_step(&g_, &pools, stage_.table() + size_t(np) * stride, stride, stage_.len(), nd, T, dk, dv,
                                  kv_dtype, dq, dq_dtype, softmax_scale, nullptr, dout, workspace_.get(), workspace_.size(),
                                  nullptr, stream_), "kv8_decode_step");
    }
  }
  void Commit() { sched_.Commit(); }

  const BatchScheduler& scheduler() const { return sched_; }
  bool idle() const { return sched_.idle(); }
  int32_t running() const { return sched_.running(); }
  int32_t queued() const { return sched_.queued(); }
  int32_t free_pages() const { return sched_.free_pages(); }
  int32_t n_layers() const { return int32_t(layers_.size()); }
  int32_t page_table_stride() const { return stage_.stride(); }
  const BatchStats& stats() const { return sched_.stats(); }
  const yahkv_geometry& geometry() const { return g_; }
  yahkv_kv8_pools pools(int32_t layer) const {
    const Layer& L = layers_.at(size_t(layer));
    return yahkv_kv8_pools{L.buf[0].get(),  L.buf[1].get(),  L.buf[2].get(),  L.buf[3].get(),  L.buf[4].get(),  L.buf[5].get(),
                           L.buf[0].size(), L.buf[1].size(), L.buf[2].size(), L.buf[3].size(), L.buf[4].size(), L.buf[5].size()};
  }
  const std::vector<int32_t>& pages(int64_t id) const { return sched_.pages(id); }
  int32_t length(int64_t id) const { return sched_.length(id); }

 private:
  struct Layer {
    DeviceBuffer buf[6];  // kq, ks, km, vq, vs, vopen
  };
  yahkv_geometry g_;
  hipStream_t stream_;
  BatchScheduler sched_;
  StepStage stage_;
  std::vector<Layer> layers_;
  DeviceBuffer workspace_, images_;
};

}  // namespace yahkv_host

#endif  // YAHKV_KV8_BATCHER_HPP_
