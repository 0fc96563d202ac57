// Host-side owner of one attention layer's paged, quantized KV cache, above the C ABI of yahkv.h.
//
// The classes keep the names and the call order of the reference's host code for this path, so that its model loop
// reads the same: LoomDecoderState -> KvDecoderState (engine/model/loom_decoder.hpp:43-51), LoomDecoder::OwnState /
// Bind / Step / ResumeAt (:159-209, 229-307), the pool byte formulas KqBytes .. VsBytes (:151-154), and the prefill's
// per-chunk order "quantize the chunk's K and V into their pages, then attend" (engine/model/loom_prefill.hpp:3341-3410).
// Host checks throw KvError where the reference throws LoomError (loom_runtime.hpp:44-60); kernels never report.
// What the reference does not have is added here: several sequences at once, and a page allocator with a free list
// (its page table is the identity, loom_decoder.hpp:175-179).
//
// Header-only, host code only; link libyahkv.so and the HIP runtime. One host thread, one stream, as the reference
// (engine/model/generator.hpp:56); stream order is the only synchronization.
#ifndef YAHKV_KV_CACHE_HPP_
#define YAHKV_KV_CACHE_HPP_

#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <memory>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "yahkv.h"

namespace yahkv_host {

class KvError : public std::runtime_error {
 public:
  using std::runtime_error::runtime_error;
};

inline void Check(int status, const char* what) {
  if (status != YAHKV_OK) throw KvError(std::string(what) + ": " + yahkv_strerror(status));
}
inline void CheckHip(hipError_t e, const char* what) {
  if (e != hipSuccess) throw KvError(std::string(what) + ": " + hipGetErrorString(e));
}

// Device allocation with its size (LoomBuffer, loom_runtime.hpp:62-89).
class DeviceBuffer {
 public:
  DeviceBuffer() = default;
  explicit DeviceBuffer(size_t bytes) : size_(bytes) { CheckHip(hipMalloc(&ptr_, bytes ? bytes : 1), "hipMalloc"); }
  DeviceBuffer(DeviceBuffer&& o) noexcept : ptr_(o.ptr_), size_(o.size_) { o.ptr_ = nullptr, o.size_ = 0; }
  DeviceBuffer& operator=(DeviceBuffer&& o) noexcept {
    std::swap(ptr_, o.ptr_), std::swap(size_, o.size_);
    return *this;
  }
  DeviceBuffer(const DeviceBuffer&) = delete;
  DeviceBuffer& operator=(const DeviceBuffer&) = delete;
  ~DeviceBuffer() {
    if (ptr_ != nullptr) (void)hipFree(ptr_);
  }
  void* get() const { return ptr_; }
  size_t size() const { return size_; }

 private:
  void* ptr_ = nullptr;
  size_t size_ = 0;
};

// A borrowed range of device memory (hrx_buffer_ref_t: buffer, offset, length).
struct BufferRef {
  void* ptr = nullptr;
  size_t length = 0;
};

// One layer's pools and the page table, owned by whoever made them; the decoder and the prefill borrow them.
struct KvDecoderState {
  BufferRef kq, ks, vq, vs;  // codes and scales of K and V (LoomDecoderState::kq/ks/vq/vs)
  BufferRef ptab;            // int32 [max_seqs][pages_per_seq]
};

// The ABI's view of a state's pools: addresses and lengths (the entry points refuse pools shorter than the geometry needs).
inline yahkv_pools PoolsOf(const KvDecoderState& st) {
  return yahkv_pools{st.kq.ptr, st.ks.ptr, st.vq.ptr, st.vs.ptr, st.kq.length, st.ks.length, st.vq.length, st.vs.length};
}

// Host page allocator with a free list (yahkv_pagepool_*).
class PagePool {
 public:
  explicit PagePool(int32_t n_pages) : p_(yahkv_pagepool_create(n_pages)) {
    if (p_ == nullptr) throw KvError("page pool: bad size");
  }
  PagePool(const PagePool&) = delete;
  PagePool& operator=(const PagePool&) = delete;
  ~PagePool() { yahkv_pagepool_destroy(p_); }
  int32_t free_count() const { return yahkv_pagepool_free_count(p_); }
  std::vector<int32_t> Alloc(int32_t n) {
    std::vector<int32_t> out(static_cast<size_t>(n));
    Check(yahkv_pagepool_alloc(p_, n, out.data()), "page pool");
    return out;
  }
  void Free(const std::vector<int32_t>& pages) {
    Check(yahkv_pagepool_free(p_, pages.data(), static_cast<int32_t>(pages.size())), "page pool");
  }
  void Shuffle(uint64_t seed) { yahkv_pagepool_shuffle(p_, seed); }
  void Retain(const std::vector<int32_t>& pages) {
    Check(yahkv_pagepool_retain(p_, pages.data(), static_cast<int32_t>(pages.size())), "page pool");
  }
  int32_t owners(int32_t page) const { return yahkv_pagepool_refcount(p_, page); }
  const yahkv_pagepool* handle() const { return p_; }

 private:
  yahkv_pagepool* p_;
};

// The decode step of one layer for a batch of sequences: append one token per active sequence, then attend.
class KvDecoder {
 public:
  // context: tokens a sequence may hold (the reference's decode.txt "ctx T", loom_decoder.hpp:64-69).
  KvDecoder(const yahkv_geometry& g, int32_t max_seqs, int32_t context, hipStream_t stream = nullptr)
      : g_(g), max_seqs_(max_seqs), T_(context), stream_(stream) {
    Check(yahkv_check_geometry(&g_), "decoder");
    if (max_seqs <= 0 || context <= 0) throw KvError("decoder: bad batch or context");
    stride_ = (context + g_.page_tokens - 1) / g_.page_tokens;
    table_.assign(size_t(max_seqs_) * stride_, 0);
    len_.assign(size_t(max_seqs_), 0);
    pages_.resize(size_t(max_seqs_));
    pos_dev_ = DeviceBuffer(sizeof(int32_t) * size_t(max_seqs_) * 2);  // [0]: positions to write, [1]: lengths to attend
    workspace_ = DeviceBuffer(yahkv_decode_workspace_bytes(&g_, max_seqs_, T_, nullptr));
    // Positions travel through pinned host memory; a step's copy may still be waiting in the stream when the next
    // step is queued, so there is a ring of staging rows, each with an event that tells when its copy has run.
    CheckHip(hipHostMalloc(reinterpret_cast<void**>(&pos_host_), sizeof(int32_t) * size_t(max_seqs_) * 2 * kStaging),
             "hipHostMalloc");
    for (auto& e : staged_) CheckHip(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
  }
  KvDecoder(const KvDecoder&) = delete;
  KvDecoder& operator=(const KvDecoder&) = delete;
  ~KvDecoder() {
    if (pos_host_ != nullptr) (void)hipHostFree(pos_host_);
    for (auto& e : staged_)
      if (e != nullptr) (void)hipEventDestroy(e);
  }

  int32_t context() const { return T_; }
  std::pair<uint32_t, uint32_t> kv_bits() const { return {uint32_t(g_.format), uint32_t(g_.format)}; }
  bool quant() const { return true; }
  size_t KqBytes() const { return yahkv_kq_bytes(&g_); }
  size_t KsBytes() const { return yahkv_ks_bytes(&g_); }
  size_t VqBytes() const { return yahkv_vq_bytes(&g_); }
  size_t VsBytes() const { return yahkv_vs_bytes(&g_); }
  int32_t page_table_stride() const { return stride_; }
  int32_t length(int32_t seq) const { return len_.at(size_t(seq)); }
  const std::vector<int32_t>& pages(int32_t seq) const { return pages_.at(size_t(seq)); }
  int32_t free_pages() const { return pool_ ? pool_->free_count() : 0; }

  // The decoder's own pools, page table and allocator (loom_decoder.hpp:159-183).
  KvDecoderState OwnState(uint64_t shuffle_seed = 0) {
    own_.clear();
    own_.emplace_back(KqBytes()), own_.emplace_back(KsBytes()), own_.emplace_back(VqBytes()), own_.emplace_back(VsBytes());
    own_.emplace_back(sizeof(int32_t) * table_.size());
    pool_.reset(new PagePool(g_.n_pages));
    if (shuffle_seed != 0) pool_->Shuffle(shuffle_seed);
    KvDecoderState st;
    st.kq = {own_[0].get(), own_[0].size()}, st.ks = {own_[1].get(), own_[1].size()};
    st.vq = {own_[2].get(), own_[2].size()}, st.vs = {own_[3].get(), own_[3].size()};
    st.ptab = {own_[4].get(), own_[4].size()};
    return st;
  }

  // External state: sizes are checked against this decoder's geometry and context (loom_decoder.hpp:186-209).
  void Bind(const KvDecoderState& st) {
    if (st.kq.ptr == nullptr || st.ks.ptr == nullptr || st.vq.ptr == nullptr || st.vs.ptr == nullptr)
      throw KvError("decoder: quantized K / V pools expected");
    if (st.kq.length < KqBytes() || st.ks.length < KsBytes() || st.vq.length < VqBytes() || st.vs.length < VsBytes())
      throw KvError("decoder: quantized KV pool smaller than the geometry's " + std::to_string(g_.n_pages) + " pages");
    if (st.ptab.ptr == nullptr || st.ptab.length < sizeof(int32_t) * table_.size())
      throw KvError("decoder: page table too small");
    st_ = st;
    bound_ = true;
    if (!pool_) pool_.reset(new PagePool(g_.n_pages));
    table_dirty_ = true;
  }

  // Pages for sequence `seq` up to `new_len` tokens; the table goes to the device before the next kernel.
  void Reserve(int32_t seq, int32_t new_len) {
    if (seq < 0 || seq >= max_seqs_) throw KvError("decoder: no such sequence");
    if (new_len > T_) throw KvError("decoder: position past the context");
    auto& pg = pages_[size_t(seq)];
    const int32_t need = (new_len + g_.page_tokens - 1) / g_.page_tokens - int32_t(pg.size());
    if (need <= 0) return;
    const std::vector<int32_t> got = pool_->Alloc(need);  // throws when the pool is exhausted
    for (int32_t p : got) {
      table_[size_t(seq) * stride_ + pg.size()] = p;
      pg.push_back(p);
    }
    table_dirty_ = true;
  }
  // Drops a sequence: its pages go back to the free list.
  void Release(int32_t seq) {
    auto& pg = pages_.at(size_t(seq));
    if (!pg.empty()) pool_->Free(pg);
    pg.clear();
    len_[size_t(seq)] = 0;
  }
  // Sequence `dst` (empty) becomes a copy of `src` that shares its full pages; the last, partly filled page is copied,
  // so both can go on appending. (The reference reuses a prefix by loading a saved slot, loom_prefill.hpp:976-1024.)
  void Fork(int32_t src, int32_t dst) {
    if (!bound_) throw KvError("decoder: no state bound");
    if (src == dst || !pages_.at(size_t(dst)).empty()) throw KvError("decoder: fork needs an empty target sequence");
    const auto& from = pages_.at(size_t(src));
    const int32_t len = len_[size_t(src)], full = len / g_.page_tokens;
    std::vector<int32_t> shared(from.begin(), from.begin() + full);
    pool_->Retain(shared);
    auto& to = pages_[size_t(dst)];
    to = shared;
    if (len % g_.page_tokens != 0) {
      const std::vector<int32_t> own = pool_->Alloc(1);
      const int32_t pair[2] = {from[size_t(full)], own[0]};
      DeviceBuffer ids(sizeof pair);
      CheckHip(hipMemcpyAsync(ids.get(), pair, sizeof pair, hipMemcpyHostToDevice, stream_), "fork");
      const yahkv_pools pools = PoolsOf(st_);
      Check(yahkv_copy_pages(&g_, &pools, static_cast<const int32_t*>(ids.get()),
                             static_cast<const int32_t*>(ids.get()) + 1, 1, stream_), "copy_pages");
      CheckHip(hipStreamSynchronize(stream_), "fork");  // `ids` and `pair` go out of scope
      to.push_back(own[0]);
    }
    for (size_t i = 0; i < to.size(); ++i) table_[size_t(dst) * stride_ + i] = to[i];
    len_[size_t(dst)] = len;
    table_dirty_ = true;
  }

  // A sequence's state as a slot file: the 64-byte header and the sequence's pages, raw (yahkv_slot_pack); LoadSlot
  // puts it into free pages of this decoder and returns the tokens it covers, so the caller continues at that
  // position (SaveState / LoadState, loom_prefill.hpp:979-1019).
  void SaveSlot(int32_t seq, const std::string& path) {
    if (!bound_) throw KvError("decoder: no state bound");
    const auto& pg = pages_.at(size_t(seq));
    const int32_t len = len_[size_t(seq)], np = (len + g_.page_tokens - 1) / g_.page_tokens;
    if (np <= 0) throw KvError("decoder: nothing to save");
    Upload();
    const size_t bytes = yahkv_slot_bytes(&g_, np);
    DeviceBuffer slot(bytes);
    const yahkv_pools pools = PoolsOf(st_);
    Check(yahkv_slot_pack(&g_, &pools, static_cast<const int32_t*>(st_.ptab.ptr) + size_t(seq) * stride_, np, len,
                          slot.get(), stream_), "slot_pack");
    std::vector<uint8_t> host(bytes);
    CheckHip(hipMemcpyAsync(host.data(), slot.get(), bytes, hipMemcpyDeviceToHost, stream_), "slot");
    CheckHip(hipStreamSynchronize(stream_), "slot");
    FILE* f = std::fopen(path.c_str(), "wb");
    if (f == nullptr) throw KvError("decoder: cannot write the slot " + path);
    const bool ok = std::fwrite(host.data(), 1, bytes, f) == bytes;
    if (std::fclose(f) != 0 || !ok) throw KvError("decoder: short write to the slot " + path);
    (void)pg;
  }
  int32_t LoadSlot(int32_t seq, const std::string& path) {
    if (!bound_) throw KvError("decoder: no state bound");
    if (!pages_.at(size_t(seq)).empty()) throw KvError("decoder: a slot loads into an empty sequence");
    FILE* f = std::fopen(path.c_str(), "rb");
    if (f == nullptr) throw KvError("decoder: cannot open the slot " + path);
    std::vector<uint8_t> host;
    uint8_t buf[1 << 16];
    for (size_t n; (n = std::fread(buf, 1, sizeof buf, f)) > 0;) host.insert(host.end(), buf, buf + n);
    std::fclose(f);
    int32_t np = 0, len = 0;
    if (yahkv_slot_check(&g_, host.data(), host.size(), &np, &len) != YAHKV_OK)
      throw KvError("decoder: the slot " + path + " does not match this geometry");
    // the header's page count is the one the tokens need, and the sequence's row holds exactly those pages: a slot
    // never reaches pages the sequence does not own
    if (np != (len + g_.page_tokens - 1) / g_.page_tokens || np > stride_)
      throw KvError("decoder: the slot " + path + " names more pages than its tokens fill");
    Reserve(seq, len);
    if (int32_t(pages_[size_t(seq)].size()) != np) throw KvError("decoder: the slot " + path + " does not fit the sequence");
    Upload();
    DeviceBuffer slot(host.size());
    CheckHip(hipMemcpyAsync(slot.get(), host.data(), host.size(), hipMemcpyHostToDevice, stream_), "slot");
    const yahkv_pools pools = PoolsOf(st_);
    Check(yahkv_slot_unpack(&g_, &pools, static_cast<const int32_t*>(st_.ptab.ptr) + size_t(seq) * stride_, np,
                            slot.get(), stream_), "slot_unpack");
    CheckHip(hipStreamSynchronize(stream_), "slot");
    len_[size_t(seq)] = len;
    return len;
  }

  // The next Step of `seq` writes position pos (after a prefill that filled positions 0 .. pos - 1; loom_decoder.hpp:145).
  void ResumeAt(int32_t seq, int32_t pos) {
    Reserve(seq, pos);
    len_.at(size_t(seq)) = pos;
  }

  // Queues one decode step for sequences 0 .. n_seqs - 1: K / V rows [n_seqs][1][H][D] of kv_dtype are appended at each
  // sequence's current length, then q [n_seqs][n_q][D] attends over the lengthened sequences into out f32.
  // What LoomDecoder::Step does in four dispatches (kappend, vappend, part, reduce: loom_decoder.hpp:253-268) takes two
  // here: the split-K pass over the tokens already in the pools, and the merge, which quantizes and stores the new
  // token and adds its term (yahkv_decode_step).
  void Step(int32_t n_seqs, const void* k, const void* v, int32_t kv_dtype, const void* q, int32_t q_dtype,
            float softmax_scale, const float* gate, float* out) {
    if (!bound_) throw KvError("decoder: no state bound");
    if (n_seqs <= 0 || n_seqs > max_seqs_) throw KvError("decoder: bad batch");
    for (int32_t s = 0; s < n_seqs; ++s)
      if (len_[size_t(s)] >= T_) throw KvError("decoder: position past the set's context");
    // the staging row of this step: free once the copy queued from it kStaging steps ago has run
    const size_t slot = step_ % kStaging;
    if (step_ >= kStaging) CheckHip(hipEventSynchronize(staged_[slot]), "positions");
    int32_t* row = pos_host_ + slot * size_t(max_seqs_) * 2;
    for (int32_t s = 0; s < n_seqs; ++s) {
      Reserve(s, len_[size_t(s)] + 1);
      row[s] = len_[size_t(s)];
      row[max_seqs_ + s] = ++len_[size_t(s)];
    }
    Upload();
    CheckHip(hipMemcpyAsync(pos_dev_.get(), row, sizeof(int32_t) * size_t(max_seqs_) * 2, hipMemcpyHostToDevice,
                            stream_), "positions");
    CheckHip(hipEventRecord(staged_[slot], stream_), "positions");
    ++step_;
    const yahkv_pools pools = PoolsOf(st_);
    const int32_t* pos = static_cast<const int32_t*>(pos_dev_.get());
    const int32_t* ptab = static_cast<const int32_t*>(st_.ptab.ptr);
    Check(yahkv_decode_step(&g_, &pools, ptab, stride_, pos + max_seqs_, n_seqs, T_, k, v, kv_dtype, q, q_dtype,
                            softmax_scale, gate, out, workspace_.get(), workspace_.size(), &opt_, stream_),
          "decode_step");
  }

  // Set-up, once a batch is in place (and again when its shape changes much): measures the XCDs' relative read speeds
  // on sequences 0 .. n_seqs - 1 as they stand and keeps them for the steps to come (yahkv_decode_calibrate; worth
  // about a percent of a large batch's step). Waits for the stream; the pools and lengths are left as they are.
  void Calibrate(int32_t n_seqs, const void* q, int32_t q_dtype, int32_t rounds = 3) {
    if (!bound_) throw KvError("decoder: no state bound");
    if (n_seqs <= 0 || n_seqs > max_seqs_) throw KvError("decoder: bad batch");
    Upload();
    std::vector<int32_t> len(size_t(max_seqs_), 0);
    for (int32_t s = 0; s < n_seqs; ++s) len[size_t(s)] = len_[size_t(s)];
    DeviceBuffer dlen(sizeof(int32_t) * size_t(max_seqs_));
    CheckHip(hipMemcpyAsync(dlen.get(), len.data(), sizeof(int32_t) * len.size(), hipMemcpyHostToDevice, stream_), "lengths");
    CheckHip(hipStreamSynchronize(stream_), "lengths");
    const yahkv_pools pools = PoolsOf(st_);
    Check(yahkv_decode_calibrate(&g_, &pools, static_cast<const int32_t*>(st_.ptab.ptr), stride_,
                                 static_cast<const int32_t*>(dlen.get()), n_seqs, T_, q, q_dtype, workspace_.get(),
                                 workspace_.size(), &opt_, rounds, stream_), "decode_calibrate");
  }
  const yahkv_decode_options& options() const { return opt_; }

  const yahkv_geometry& geometry() const { return g_; }
  const KvDecoderState& state() const { return st_; }
  hipStream_t stream() const { return stream_; }
  // Validates and uploads the page table if it changed (loom_prefill.hpp:1306-1319).
  void Upload() {
    if (!table_dirty_) return;
    Check(yahkv_validate_shared_page_table(&g_, pool_->handle(), table_.data(), stride_, PagesAsLengths().data(),
                                           max_seqs_), "page table");
    CheckHip(hipMemcpyAsync(st_.ptab.ptr, table_.data(), sizeof(int32_t) * table_.size(), hipMemcpyHostToDevice, stream_),
             "page table upload");
    // the host table may be edited again only after this copy has run
    CheckHip(hipStreamSynchronize(stream_), "page table upload");
    table_dirty_ = false;
  }
  void SetLength(int32_t seq, int32_t len) { len_.at(size_t(seq)) = len; }

 private:
  std::vector<int32_t> PagesAsLengths() const {  // validate every page a sequence owns
    std::vector<int32_t> v(static_cast<size_t>(max_seqs_), 0);
    for (int32_t s = 0; s < max_seqs_; ++s) v[size_t(s)] = int32_t(pages_[size_t(s)].size()) * g_.page_tokens;
    return v;
  }

  yahkv_geometry g_;
  int32_t max_seqs_, T_, stride_ = 0;
  hipStream_t stream_;
  std::vector<int32_t> table_, len_;
  std::vector<std::vector<int32_t>> pages_;
  std::vector<DeviceBuffer> own_;
  std::unique_ptr<PagePool> pool_;
  DeviceBuffer pos_dev_, workspace_;
  yahkv_decode_options opt_{};  // defaults, and the XCD shares once Calibrate has run
  static constexpr size_t kStaging = 4;
  int32_t* pos_host_ = nullptr;  // [kStaging][2][max_seqs]
  hipEvent_t staged_[kStaging] = {nullptr, nullptr, nullptr, nullptr};
  size_t step_ = 0;
  KvDecoderState st_;
  bool bound_ = false, table_dirty_ = true;
};

// Chunked prefill of one layer on the decoder's state: quantize the chunk into newly reserved pages, then causal
// attention of the chunk's queries over prefix + chunk (loom_prefill.hpp:3341-3410: kq / vq, then the attention).
class KvPrefill {
 public:
  explicit KvPrefill(KvDecoder& dec) : dec_(dec), prefix_dev_(sizeof(int32_t) * 1024) {}

  // Sequences 0 .. n_seqs - 1 each take `chunk_len` more tokens: k / v [n_seqs][chunk_len][H][D] of kv_dtype,
  // q [n_seqs][chunk_len][n_q][D] bf16, out of out_dtype. Afterwards the decoder continues at the new lengths
  // (DecoderState + ResumeAt in the reference, loom_prefill.hpp:950-970, engine.hpp:203).
  void RunChunk(int32_t n_seqs, int32_t chunk_len, const void* k, const void* v, int32_t kv_dtype, const void* q,
                float softmax_scale, const float* gate, void* out, int32_t out_dtype) {
    if (n_seqs <= 0 || n_seqs > 1024) throw KvError("prefill: bad batch");
    std::vector<int32_t> prefix(static_cast<size_t>(n_seqs));
    int32_t max_prefix = 0;
    for (int32_t s = 0; s < n_seqs; ++s) {
      prefix[size_t(s)] = dec_.length(s);
      max_prefix = std::max(max_prefix, prefix[size_t(s)]);
      dec_.Reserve(s, prefix[size_t(s)] + chunk_len);
    }
    dec_.Upload();
    CheckHip(hipMemcpyAsync(prefix_dev_.get(), prefix.data(), sizeof(int32_t) * prefix.size(), hipMemcpyHostToDevice,
                            dec_.stream()), "prefix lengths");
    CheckHip(hipStreamSynchronize(dec_.stream()), "prefix lengths");  // `prefix` is a local
    const KvDecoderState& st = dec_.state();
    const yahkv_pools pools = PoolsOf(st);
    const int32_t* ptab = static_cast<const int32_t*>(st.ptab.ptr);
    const int32_t* pre = static_cast<const int32_t*>(prefix_dev_.get());
    Check(yahkv_append(&dec_.geometry(), &pools, ptab, dec_.page_table_stride(), pre, nullptr, n_seqs, chunk_len, k, v,
                       kv_dtype, dec_.stream()), "append");
    // the decoded prefix (bf16 tile images) lives in a buffer that grows with the longest call so far
    const size_t need = yahkv_prefill_workspace_bytes(&dec_.geometry(), n_seqs, max_prefix, chunk_len);
    if (need > images_.size()) {
      CheckHip(hipStreamSynchronize(dec_.stream()), "prefill workspace");
      images_ = DeviceBuffer(need);
    }
    Check(yahkv_prefill_attend(&dec_.geometry(), &pools, ptab, dec_.page_table_stride(), pre, n_seqs, max_prefix,
                               chunk_len, q, softmax_scale, gate, out, out_dtype, images_.get(), images_.size(),
                               dec_.stream()), "prefill_attend");
    for (int32_t s = 0; s < n_seqs; ++s) dec_.SetLength(s, prefix[size_t(s)] + chunk_len);
  }

 private:
  KvDecoder& dec_;
  DeviceBuffer prefix_dev_, images_;
};

}  // namespace yahkv_host

#endif  // YAHKV_KV_CACHE_HPP_
