// Continuous batching over the paged, quantized KV cache, above the C ABI of yahkv.h.
//
// The reference serves one sequence at a time: TextGenerator::Generate runs the prompt in chunks through the prefill,
// then one decode step per token, and is not reentrant (engine/model/generator.hpp:48-59, engine/model/engine.hpp:
// 123-250). With a page allocator many requests can share the pools, and these classes are the step loop that does
// it: requests wait in a queue, are admitted while pages last, take their prompt in chunks (the reference's prefill
// chunk, engine.hpp:147-170) next to the requests that are already decoding, and give their pages back when they
// end. When the pool runs out in the middle of a step the request admitted last is put back into the queue and starts
// again from its first token (its pages are the cheapest to lose).
//
// BatchScheduler is the bookkeeping alone (queue, pages, plan): host code with no GPU call in it. KvBatcher adds the
// pools of the attention layers (one page table serves all layers, as in the reference, loom_decoder.hpp:175-179) and
// runs a planned step layer by layer. The model around it (embedding, projections, sampling) is the caller's:
//   const BatchPlan& plan = b.Schedule();        // which request takes which positions
//   for (layer ...) {
//     ... the caller computes this layer's K, V and Q rows for exactly those positions, in the plan's order ...
//     b.RunLayer(layer, ...);                    // append + attention for the whole plan
//   }
//   b.Commit();                                  // the positions are done
//   for (int64_t id : b.TakeFinished()) ...      // their pages are free again
//
// Header-only, host code only; one host thread, one stream (generator.hpp:56).
#ifndef YAHKV_KV_BATCHER_HPP_
#define YAHKV_KV_BATCHER_HPP_

#include <deque>
#include <map>

#include "kv_cache.hpp"

namespace yahkv_host {

// Tokens [pos, pos + n) of request `id`: a prompt chunk (n <= chunk) or one decode token (n == 1).
struct BatchWork {
  int64_t id;
  int32_t pos, n;
};
struct BatchPlan {
  std::vector<BatchWork> prefill, decode;
  bool empty() const { return prefill.empty() && decode.empty(); }
};
struct BatchStats {
  int64_t steps = 0, prefill_tokens = 0, decode_tokens = 0, admitted = 0, preempted = 0, finished = 0;
  int32_t peak_running = 0, peak_pages = 0;
};

class BatchScheduler {
 public:
  // n_pages of page_tokens tokens each; max_running: requests that hold pages at once; context: tokens a request may
  // hold (prompt + generated); chunk: prompt tokens a request takes per step; max_prefill: requests that take a
  // prompt chunk in the same step.
  BatchScheduler(int32_t n_pages, int32_t page_tokens, int32_t max_running, int32_t context, int32_t chunk,
                 int32_t max_prefill, uint64_t shuffle_seed = 0)
      : n_pages_(n_pages), pt_(page_tokens), max_running_(max_running), T_(context), chunk_(chunk),
        max_prefill_(max_prefill), pool_(n_pages) {
    if (page_tokens <= 0 || max_running <= 0 || context <= 0 || chunk <= 0 || max_prefill <= 0 || max_prefill > max_running)
      throw KvError("batcher: bad sizes");
    if (shuffle_seed != 0) pool_.Shuffle(shuffle_seed);
  }

  // A request of prompt_len prompt tokens that then appends max_new generated tokens: positions 0 .. prompt_len +
  // max_new - 1. Refused when it could never run: longer than the context or than the whole pool.
  void Submit(int64_t id, int32_t prompt_len, int32_t max_new) {
    if (prompt_len <= 0 || max_new < 0) throw KvError("batcher: bad request");
    if (int64_t(prompt_len) + max_new > T_) throw KvError("batcher: request longer than the context");
    if (Pages(prompt_len + max_new) > n_pages_) throw KvError("batcher: request larger than the pool");
    if (req_.count(id) != 0) throw KvError("batcher: request id in use");
    req_[id] = Request{prompt_len, max_new};
    queue_.push_back(id);
  }

  // Ends a request early (a stop token, a client that went away): it takes no further work and its pages come back
  // with the next TakeFinished.
  void Stop(int64_t id) {
    if (planned_) throw KvError("batcher: Stop between Schedule and Commit");
    auto it = req_.find(id);
    if (it == req_.end() || it->second.state == kDone) return;
    if (it->second.state == kQueued) queue_.erase(std::find(queue_.begin(), queue_.end(), id));
    if (it->second.state == kRunning) running_.erase(std::find(running_.begin(), running_.end(), id));
    it->second.state = kDone;
    done_.push_back(id);
  }

  // Plans the next step and reserves its pages. Running requests come first, in the order they were admitted: those
  // past their prompt take one decode token each, up to max_prefill of the others a prompt chunk. When the pool cannot
  // hold that, the request admitted last goes back to the head of the queue. Then queued requests are admitted, in
  // order, while a slot, a place among the step's chunks and the pages of their first chunk are free (plus one page
  // of slack per running request, so that an admission is not undone by the next decode step).
  const BatchPlan& Schedule() {
    if (planned_) throw KvError("batcher: Schedule twice without Commit");
    Reap();
    plan_.prefill.clear(), plan_.decode.clear();
    const int64_t preempted_before = stats_.preempted;
    for (int64_t id : running_) Plan(id);
    for (bool again = true; again;) {
      again = false;
      for (const std::vector<BatchWork>* list : {&plan_.decode, &plan_.prefill}) {
        for (const BatchWork& w : *list) {
          if (Reserve(req_[w.id], w.pos + w.n)) continue;
          if (running_.size() <= 1) throw KvError("batcher: the pool cannot hold one request");
          Preempt(running_.back());
          again = true;
          break;
        }
        if (again) break;
      }
    }
    while (!queue_.empty() && int32_t(running_.size()) < max_running_ && int32_t(plan_.prefill.size()) < max_prefill_ &&
           stats_.preempted == preempted_before) {  // a step that had to put a request back admits nobody
      const int64_t id = queue_.front();
      Request& r = req_[id];
      const int32_t first = std::min(chunk_, r.prompt);
      if (pool_.free_count() < Pages(first) + int32_t(running_.size())) break;
      queue_.pop_front();
      r.state = kRunning, r.done = 0;
      running_.push_back(id);
      ++stats_.admitted;
      Plan(id);
      Reserve(r, first);
    }
    stats_.peak_running = std::max(stats_.peak_running, int32_t(running_.size()));
    stats_.peak_pages = std::max(stats_.peak_pages, n_pages_ - pool_.free_count());
    planned_ = true;
    return plan_;
  }

  // The planned positions are done (their K and V are in the pages): requests advance, those at their end stop.
  void Commit() {
    if (!planned_) throw KvError("batcher: Commit without Schedule");
    planned_ = false;
    if (plan_.empty()) return;
    for (const std::vector<BatchWork>* list : {&plan_.prefill, &plan_.decode}) {
      for (const BatchWork& w : *list) {
        Request& r = req_[w.id];
        r.done = w.pos + w.n;
        if (r.done >= r.prompt + r.max_new) {
          running_.erase(std::find(running_.begin(), running_.end(), w.id));
          r.state = kDone;
          done_.push_back(w.id);
        }
      }
    }
    ++stats_.steps;
    for (const BatchWork& w : plan_.prefill) stats_.prefill_tokens += w.n;
    stats_.decode_tokens += int64_t(plan_.decode.size());
  }

  // Requests that ended since the last call; their pages return to the free list here. (Kernels still reading them
  // were queued before anything that will write them again, and the one stream keeps that order.)
  std::vector<int64_t> TakeFinished() {
    std::vector<int64_t> out = done_;
    Reap();
    return out;
  }

  bool idle() const { return queue_.empty() && running_.empty(); }
  bool planned() const { return planned_; }
  const BatchPlan& plan() const { return plan_; }
  int32_t running() const { return int32_t(running_.size()); }
  int32_t queued() const { return int32_t(queue_.size()); }
  int32_t free_pages() const { return pool_.free_count(); }
  int32_t n_pages() const { return n_pages_; }
  int32_t chunk() const { return chunk_; }
  int32_t context() const { return T_; }
  int32_t max_running() const { return max_running_; }
  int32_t max_prefill() const { return max_prefill_; }
  const BatchStats& stats() const { return stats_; }
  const PagePool& pool() const { return pool_; }
  // Pages and length of a request that holds pages (running, or ended and not yet taken).
  const std::vector<int32_t>& pages(int64_t id) const { return req_.at(id).pages; }
  int32_t length(int64_t id) const { return req_.at(id).done; }
  // Ids that hold pages: the running requests in the order of admission, then those that ended and were not taken.
  std::vector<int64_t> holders() const {
    std::vector<int64_t> v = running_;
    v.insert(v.end(), done_.begin(), done_.end());
    return v;
  }
  // Ids that wait, in the order they will be admitted.
  std::vector<int64_t> waiting() const { return std::vector<int64_t>(queue_.begin(), queue_.end()); }

 private:
  enum State { kQueued, kRunning, kDone };
  struct Request {
    int32_t prompt = 0, max_new = 0;
    int32_t done = 0;  // positions whose K and V are in the pages
    State state = kQueued;
    std::vector<int32_t> pages;
  };

  int32_t Pages(int32_t tokens) const { return (tokens + pt_ - 1) / pt_; }
  void Plan(int64_t id) {
    const Request& r = req_[id];
    if (r.done >= r.prompt) {
      plan_.decode.push_back(BatchWork{id, r.done, 1});
    } else if (int32_t(plan_.prefill.size()) < max_prefill_) {
      plan_.prefill.push_back(BatchWork{id, r.done, std::min(chunk_, r.prompt - r.done)});
    }
  }
  bool Reserve(Request& r, int32_t new_len) {
    const int32_t need = Pages(new_len) - int32_t(r.pages.size());
    if (need <= 0) return true;
    if (pool_.free_count() < need) return false;
    const std::vector<int32_t> got = pool_.Alloc(need);
    r.pages.insert(r.pages.end(), got.begin(), got.end());
    return true;
  }
  void Preempt(int64_t id) {
    Request& r = req_[id];
    // Kernels of earlier steps may still be reading these pages; they were queued before anything that will write
    // them again, and stream order keeps that.
    if (!r.pages.empty()) pool_.Free(r.pages);
    r.pages.clear();
    r.done = 0, r.state = kQueued;
    running_.erase(std::find(running_.begin(), running_.end(), id));
    queue_.push_front(id);
    auto drop = [&](std::vector<BatchWork>& v) {
      v.erase(std::remove_if(v.begin(), v.end(), [&](const BatchWork& w) { return w.id == id; }), v.end());
    };
    drop(plan_.prefill), drop(plan_.decode);
    ++stats_.preempted;
  }
  void Reap() {
    for (int64_t id : done_) {
      Request& r = req_[id];
      if (!r.pages.empty()) pool_.Free(r.pages);
      req_.erase(id);
      ++stats_.finished;
    }
    done_.clear();
  }

  int32_t n_pages_, pt_, max_running_, T_, chunk_, max_prefill_;
  PagePool pool_;
  std::map<int64_t, Request> req_;
  std::deque<int64_t> queue_;
  std::vector<int64_t> running_, done_;  // running_: in the order of admission
  BatchPlan plan_;
  BatchStats stats_;
  bool planned_ = false;
};

// The planned step's page-table rows and columns on the device: rows of the plan's prompt chunks, then of its decode
// tokens, and per row the prefix, valid, position and length columns. Shared by the batchers of both format families.
class StepStage {
 public:
  StepStage(const yahkv_geometry& g, int32_t max_running, int32_t max_prefill, int32_t context, hipStream_t stream)
      : g_(g), stream_(stream) {
    stride_ = (context + g_.page_tokens - 1) / g_.page_tokens;
    rows_ = size_t(max_running) + size_t(max_prefill);
    ints_ = rows_ * size_t(stride_) + 4 * rows_;
    dev_ = DeviceBuffer(sizeof(int32_t) * ints_);
    CheckHip(hipHostMalloc(reinterpret_cast<void**>(&host_), sizeof(int32_t) * ints_), "hipHostMalloc");
  }
  StepStage(const StepStage&) = delete;
  StepStage& operator=(const StepStage&) = delete;
  ~StepStage() {
    if (host_ != nullptr) (void)hipHostFree(host_);
  }

  // Checks the page table the plan implies and sends it to the device.
  void Upload(const BatchScheduler& sched, const BatchPlan& plan) {
    const int32_t np = int32_t(plan.prefill.size()), nd = int32_t(plan.decode.size());
    CheckHip(hipStreamSynchronize(stream_), "batcher");  // the last step has read the staging buffer
    int32_t* table = host_;
    int32_t* prefix = host_ + rows_ * size_t(stride_);
    int32_t *valid = prefix + rows_, *pos = valid + rows_, *len = pos + rows_;
    std::vector<int32_t> owned(size_t(np + nd));
    max_prefix_ = 0;
    for (int32_t i = 0; i < np + nd; ++i) {
      const BatchWork& w = i < np ? plan.prefill[size_t(i)] : plan.decode[size_t(i - np)];
      const std::vector<int32_t>& pages = sched.pages(w.id);
      std::fill(table + size_t(i) * stride_, table + size_t(i + 1) * stride_, 0);
      std::copy(pages.begin(), pages.end(), table + size_t(i) * stride_);
      owned[size_t(i)] = int32_t(pages.size()) * g_.page_tokens;
      if (i < np) {
        prefix[i] = w.pos, valid[i] = w.n;
        max_prefix_ = std::max(max_prefix_, w.pos);
      } else {
        pos[i - np] = w.pos, len[i - np] = w.pos + 1;
      }
    }
    Check(yahkv_validate_shared_page_table(&g_, sched.pool().handle(), table, stride_, owned.data(), np + nd),
          "page table");
    CheckHip(hipMemcpyAsync(dev_.get(), host_, sizeof(int32_t) * ints_, hipMemcpyHostToDevice, stream_), "batcher upload");
  }

  int32_t stride() const { return stride_; }
  int32_t max_prefix() const { return max_prefix_; }
  // device pointers: the table's rows (prompt chunks first), the chunks' prefix lengths and valid rows, the decode
  // rows' positions and lengths
  const int32_t* table() const { return static_cast<const int32_t*>(dev_.get()); }
  const int32_t* prefix() const { return table() + rows_ * size_t(stride_); }
  const int32_t* valid() const { return prefix() + rows_; }
  const int32_t* pos() const { return valid() + rows_; }
  const int32_t* len() const { return pos() + rows_; }

 private:
  yahkv_geometry g_;
  hipStream_t stream_;
  int32_t stride_ = 0, max_prefix_ = 0;
  size_t rows_ = 0, ints_ = 0;
  DeviceBuffer dev_;
  int32_t* host_ = nullptr;
};

class KvBatcher {
 public:
  // g.n_pages pages per layer; the layers share the page table.
  KvBatcher(const yahkv_geometry& g, int32_t n_layers, int32_t max_running, int32_t context, int32_t chunk,
            int32_t max_prefill, hipStream_t stream = nullptr, uint64_t shuffle_seed = 0)
      : g_(g), stream_(stream),
        sched_(g.n_pages, g.page_tokens, max_running, context, chunk, max_prefill, shuffle_seed),
        stage_(g, max_running, max_prefill, context, stream) {
    Check(yahkv_check_geometry(&g_), "batcher");
    if (n_layers <= 0) throw KvError("batcher: bad sizes");
    for (int32_t l = 0; l < n_layers; ++l) {
      layers_.emplace_back();
      Layer& L = layers_.back();
      L.kq = DeviceBuffer(yahkv_kq_bytes(&g_)), L.ks = DeviceBuffer(yahkv_ks_bytes(&g_));
      L.vq = DeviceBuffer(yahkv_vq_bytes(&g_)), L.vs = DeviceBuffer(yahkv_vs_bytes(&g_));
    }
    workspace_ = DeviceBuffer(yahkv_decode_workspace_bytes(&g_, max_running, context, nullptr));
  }
  KvBatcher(const KvBatcher&) = delete;
  KvBatcher& operator=(const KvBatcher&) = delete;

  void Submit(int64_t id, int32_t prompt_len, int32_t max_new) { sched_.Submit(id, prompt_len, max_new); }
  void Stop(int64_t id) { sched_.Stop(id); }
  std::vector<int64_t> TakeFinished() { return sched_.TakeFinished(); }

  // Plans the step (BatchScheduler::Schedule), checks the page table it implies and sends it to the device.
  const BatchPlan& Schedule() {
    const BatchPlan& plan = sched_.Schedule();
    if (!plan.empty()) stage_.Upload(sched_, plan);
    return plan;
  }

  // Runs the planned step for one layer on the stream. Rows are in the plan's order:
  //   prompt chunks: pk, pv [n_prefill][chunk][n_kv][D] of kv_dtype, pq [n_prefill][chunk][n_q][D] bf16,
  //                  pout [n_prefill][chunk][n_q][D] of pout_dtype; rows past a chunk's n are ignored / undefined
  //   decode tokens: dk, dv [n_decode][1][n_kv][D] of kv_dtype, dq [n_decode][n_q][D] of dq_dtype, dout f32
  // Per chunk: quantize into the pages, then causal attention over prefix + chunk (loom_prefill.hpp:3341-3410); per
  // decode token: append, part, reduce (loom_decoder.hpp:253-268).
  void RunLayer(int32_t layer, const void* pk, const void* pv, const void* pq, void* pout, int32_t pout_dtype,
                const void* dk, const void* dv, const void* dq, int32_t dq_dtype, float* dout, int32_t kv_dtype,
                float softmax_scale) {
    if (!sched_.planned()) throw KvError("batcher: RunLayer without Schedule");
    if (layer < 0 || layer >= int32_t(layers_.size())) throw KvError("batcher: no such layer");
    const BatchPlan& plan = sched_.plan();
    const int32_t np = int32_t(plan.prefill.size()), nd = int32_t(plan.decode.size());
    if (np + nd == 0) return;
    const int32_t *d = stage_.table(), *d_prefix = stage_.prefix(), *d_valid = stage_.valid(), *d_len = stage_.len();
    const int32_t stride_ = stage_.stride(), max_prefix_ = stage_.max_prefix();
    const yahkv_pools pools = this->pools(layer);
    const int32_t chunk = sched_.chunk(), T = sched_.context();
    if (np > 0) {
      if (pk == nullptr || pv == nullptr || pq == nullptr || pout == nullptr) throw KvError("batcher: prompt rows missing");
      Check(yahkv_append(&g_, &pools, d, stride_, d_prefix, d_valid, np, chunk, pk, pv, kv_dtype, stream_), "append");
      const size_t need = yahkv_prefill_workspace_bytes(&g_, np, max_prefix_, chunk);
      if (need > images_.size()) {
        CheckHip(hipStreamSynchronize(stream_), "prefill workspace");
        images_ = DeviceBuffer(need);
      }
      Check(yahkv_prefill_attend(&g_, &pools, d, stride_, d_prefix, np, max_prefix_, chunk, pq, softmax_scale, nullptr,
                                 pout, pout_dtype, images_.get(), images_.size(), stream_), "prefill_attend");
    }
    if (nd > 0) {
      if (dk == nullptr || dv == nullptr || dq == nullptr || dout == nullptr) throw KvError("batcher: decode rows missing");
      const int32_t* dt = d + size_t(np) * stride_;
      // append + attention of the decode rows in two dispatches (the merge stores the new tokens)
      Check(yahkv_decode_step(&g_, &pools, dt, stride_, d_len, nd, T, dk, dv, kv_dtype, dq, dq_dtype, softmax_scale,
                              nullptr, dout, workspace_.get(), workspace_.size(), nullptr, stream_), "decode_step");
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
  yahkv_pools pools(int32_t layer) const {
    const Layer& L = layers_.at(size_t(layer));
    return yahkv_pools{L.kq.get(), L.ks.get(), L.vq.get(), L.vs.get(), L.kq.size(), L.ks.size(), L.vq.size(), L.vs.size()};
  }
  const std::vector<int32_t>& pages(int64_t id) const { return sched_.pages(id); }
  int32_t length(int64_t id) const { return sched_.length(id); }

 private:
  struct Layer {
    DeviceBuffer kq, ks, vq, vs;
  };
  yahkv_geometry g_;
  hipStream_t stream_;
  BatchScheduler sched_;
  StepStage stage_;
  std::vector<Layer> layers_;
  DeviceBuffer workspace_, images_;
};

}  // namespace yahkv_host

#endif  // YAHKV_KV_BATCHER_HPP_
