// Host-side owner of one attention layer's KV cache in the reference's own format, kv8a16, above the yahkv_kv8_* entry
// points of yahkv.h: the counterpart of kv_cache.hpp for that format.
//
// Names and call order follow the reference's host code at "kv q 8 8": LoomDecoderState {kq, ks, km, vq, vs, vopen, ptab}
// (engine/model/loom_decoder.hpp:43-51), LoomDecoder::OwnState / Bind / Step / ResumeAt (:159-209, 229-307) with its rule
// that steps over quantized V must be contiguous from a 16-key boundary unless the open tile has been seeded
// (:233-235), and the prefill's per-chunk order: channel means on the first chunk only, quantize the chunk's K and V,
// seed the open tile, attend (engine/model/loom_prefill.hpp:3343-3410, 944-947). Several sequences at once, each with
// its own means and open tile (they live with the sequence's first and newest page), and a page allocator, which the
// reference does not have.
//
// Header-only, host code only; link libyahkv.so and the HIP runtime. One host thread, one stream.
#ifndef YAHKV_KV8_CACHE_HPP_
#define YAHKV_KV8_CACHE_HPP_

#include "kv_cache.hpp"

namespace yahkv_host {

struct Kv8DecoderState {
  BufferRef kq, ks, km, vq, vs, vopen;
  BufferRef ptab;  // int32 [max_seqs][pages_per_seq]
};
inline yahkv_kv8_pools PoolsOf(const Kv8DecoderState& st) {
  return yahkv_kv8_pools{st.kq.ptr,    st.ks.ptr,    st.km.ptr,    st.vq.ptr,    st.vs.ptr,    st.vopen.ptr,
                         st.kq.length, st.ks.length, st.km.length, st.vq.length, st.vs.length, st.vopen.length};
}

class Kv8Decoder {
 public:
  Kv8Decoder(const yahkv_geometry& g, int32_t max_seqs, int32_t context, hipStream_t stream = nullptr)
      : g_(g), max_seqs_(max_seqs), T_(context), stream_(stream) {
    if (yahkv_kv8_kq_bytes(&g_) == 0) throw KvError("kv8 decoder: not a kv8a16 geometry (head_dim 256, 256-token pages)");
    if (max_seqs <= 0 || context <= 0) throw KvError("kv8 decoder: bad batch or context");
    stride_ = (context + g_.page_tokens - 1) / g_.page_tokens;
    table_.assign(size_t(max_seqs_) * stride_, 0);
    len_.assign(size_t(max_seqs_), 0);
    open_at_.assign(size_t(max_seqs_), 0);
    pages_.resize(size_t(max_seqs_));
    len_dev_ = DeviceBuffer(sizeof(int32_t) * size_t(max_seqs_));
    workspace_ = DeviceBuffer(yahkv_kv8_decode_workspace_bytes(&g_, max_seqs_, T_, nullptr));
    CheckHip(hipHostMalloc(reinterpret_cast<void**>(&len_host_), sizeof(int32_t) * size_t(max_seqs_) * kStaging), "hipHostMalloc");
    for (auto& e : staged_) CheckHip(hipEventCreateWithFlags(&e, hipEventDisableTiming), "hipEventCreate");
  }
  Kv8Decoder(const Kv8Decoder&) = delete;
  Kv8Decoder& operator=(const Kv8Decoder&) = delete;
  ~Kv8Decoder() {
    if (len_host_ != nullptr) (void)hipHostFree(len_host_);
    for (auto& e : staged_)
      if (e != nullptr) (void)hipEventDestroy(e);
  }

  int32_t context() const { return T_; }
  std::pair<uint32_t, uint32_t> kv_bits() const {
    switch (g_.format) {
      case YAHKV_KV4A16: return {4u, 4u};
      case YAHKV_K8V4A16: return {8u, 4u};
      case YAHKV_K4V8A16: return {4u, 8u};
      default: return {8u, 8u};
    }
  }
  bool quant() const { return true; }
  size_t KqBytes() const { return yahkv_kv8_kq_bytes(&g_); }
  size_t KsBytes() const { return yahkv_kv8_ks_bytes(&g_); }
  size_t VqBytes() const { return yahkv_kv8_vq_bytes(&g_); }
  size_t VsBytes() const { return yahkv_kv8_vs_bytes(&g_); }
  int32_t page_table_stride() const { return stride_; }
  int32_t length(int32_t seq) const { return len_.at(size_t(seq)); }
  const std::vector<int32_t>& pages(int32_t seq) const { return pages_.at(size_t(seq)); }
  int32_t free_pages() const { return pool_ ? pool_->free_count() : 0; }
  const yahkv_geometry& geometry() const { return g_; }
  const Kv8DecoderState& state() const { return st_; }
  hipStream_t stream() const { return stream_; }

  // The decoder's own buffers, page table and allocator (loom_decoder.hpp:159-183).
  Kv8DecoderState OwnState(uint64_t shuffle_seed = 0) {
    own_.clear();
    own_.emplace_back(KqBytes()), own_.emplace_back(KsBytes()), own_.emplace_back(yahkv_kv8_km_bytes(&g_));
    own_.emplace_back(VqBytes()), own_.emplace_back(VsBytes()), own_.emplace_back(yahkv_kv8_vopen_bytes(&g_));
    own_.emplace_back(sizeof(int32_t) * table_.size());
    pool_.reset(new PagePool(g_.n_pages));
    if (shuffle_seed != 0) pool_->Shuffle(shuffle_seed);
    Kv8DecoderState st;
    BufferRef* refs[7] = {&st.kq, &st.ks, &st.km, &st.vq, &st.vs, &st.vopen, &st.ptab};
    for (int i = 0; i < 7; ++i) *refs[i] = {own_[size_t(i)].get(), own_[size_t(i)].size()};
    return st;
  }

  // External state: sizes are checked against this decoder's geometry and context (loom_decoder.hpp:186-209).
  void Bind(const Kv8DecoderState& st) {
    const BufferRef* refs[6] = {&st.kq, &st.ks, &st.km, &st.vq, &st.vs, &st.vopen};
    const size_t need[6] = {KqBytes(), KsBytes(), yahkv_kv8_km_bytes(&g_), VqBytes(), VsBytes(), yahkv_kv8_vopen_bytes(&g_)};
    for (int i = 0; i < 6; ++i) {
      if (refs[i]->ptr == nullptr) throw KvError("kv8 decoder: quantized K / V buffers expected");
      if (refs[i]->length < need[i])
        throw KvError("kv8 decoder: a KV buffer is smaller than the geometry's " + std::to_string(g_.n_pages) + " pages");
    }
    if (st.ptab.ptr == nullptr || st.ptab.length < sizeof(int32_t) * table_.size())
      throw KvError("kv8 decoder: page table too small");
    st_ = st;
    bound_ = true;
    if (!pool_) pool_.reset(new PagePool(g_.n_pages));
    table_dirty_ = true;
  }

  // Pages for sequence `seq` up to `new_len` tokens. A sequence's first page carries its channel means: they start at
  // zero (a sequence that begins with decode steps has none, as a fresh LoomDecoderState's km, loom_decoder.hpp:168).
  void Reserve(int32_t seq, int32_t new_len) {
    if (!bound_) throw KvError("kv8 decoder: no state bound");
    if (seq < 0 || seq >= max_seqs_) throw KvError("kv8 decoder: no such sequence");
    if (new_len > T_) throw KvError("kv8 decoder: position past the context");
    auto& pg = pages_[size_t(seq)];
    const int32_t need = (new_len + g_.page_tokens - 1) / g_.page_tokens - int32_t(pg.size());
    if (need <= 0) return;
    const std::vector<int32_t> got = pool_->Alloc(need);
    for (int32_t p : got) {
      if (pg.empty()) {
        const size_t row = size_t(g_.n_kv_heads) * 256 * sizeof(float);
        CheckHip(hipMemsetAsync(static_cast<char*>(st_.km.ptr) + size_t(p) * row, 0, row, stream_), "channel means");
      }
      table_[size_t(seq) * stride_ + pg.size()] = p;
      pg.push_back(p);
    }
    table_dirty_ = true;
  }
  void Release(int32_t seq) {
    auto& pg = pages_.at(size_t(seq));
    if (!pg.empty()) pool_->Free(pg);
    pg.clear();
    len_[size_t(seq)] = 0, open_at_[size_t(seq)] = 0;
  }

  // Sequence `dst` (empty) becomes a copy of `src` that shares its full pages; the last, partly filled page is copied
  // with its open tile (and, where it is also the first page, the channel means), so both can go on appending. The
  // means of a longer sequence stay with the shared first page: they are written by the first chunk only.
  void Fork(int32_t src, int32_t dst) {
    if (!bound_) throw KvError("kv8 decoder: no state bound");
    if (src == dst || !pages_.at(size_t(dst)).empty()) throw KvError("kv8 decoder: fork needs an empty target sequence");
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
      const yahkv_kv8_pools pools = PoolsOf(st_);
      Check(yahkv_kv8_copy_pages(&g_, &pools, static_cast<const int32_t*>(ids.get()),
                                 static_cast<const int32_t*>(ids.get()) + 1, 1, stream_), "kv8_copy_pages");
      CheckHip(hipStreamSynchronize(stream_), "fork");  // `ids` and `pair` go out of scope
      to.push_back(own[0]);
    }
    for (size_t i = 0; i < to.size(); ++i) table_[size_t(dst) * stride_ + i] = to[i];
    len_[size_t(dst)] = len;
    open_at_[size_t(dst)] = open_at_[size_t(src)];
    table_dirty_ = true;
  }

  // A sequence's state as a slot file: the 64-byte header and the sequence's share of the six buffers, raw
  // (yahkv_kv8_slot_pack); LoadSlot puts it into free pages of this decoder and returns the tokens it covers, so the
  // caller continues at that position, open tile included (SaveState / LoadState, loom_prefill.hpp:979-1019).
  void SaveSlot(int32_t seq, const std::string& path) {
    if (!bound_) throw KvError("kv8 decoder: no state bound");
    const int32_t len = len_.at(size_t(seq)), np = (len + g_.page_tokens - 1) / g_.page_tokens;
    if (np <= 0) throw KvError("kv8 decoder: nothing to save");
    if (len % 16 != 0 && len != open_at_[size_t(seq)]) throw KvError("kv8 decoder: the open tile does not reach the length");
    Upload();
    const size_t bytes = yahkv_kv8_slot_bytes(&g_, np);
    DeviceBuffer slot(bytes);
    const yahkv_kv8_pools pools = PoolsOf(st_);
    Check(yahkv_kv8_slot_pack(&g_, &pools, static_cast<const int32_t*>(st_.ptab.ptr) + size_t(seq) * stride_, np, len,
                              slot.get(), stream_), "kv8_slot_pack");
    std::vector<uint8_t> host(bytes);
    CheckHip(hipMemcpyAsync(host.data(), slot.get(), bytes, hipMemcpyDeviceToHost, stream_), "slot");
    CheckHip(hipStreamSynchronize(stream_), "slot");
    FILE* f = std::fopen(path.c_str(), "wb");
    if (f == nullptr) throw KvError("kv8 decoder: cannot write the slot " + path);
    const bool ok = std::fwrite(host.data(), 1, bytes, f) == bytes;
    if (std::fclose(f) != 0 || !ok) throw KvError("kv8 decoder: short write to the slot " + path);
  }
  int32_t LoadSlot(int32_t seq, const std::string& path) {
    if (!bound_) throw KvError("kv8 decoder: no state bound");
    if (!pages_.at(size_t(seq)).empty()) throw KvError("kv8 decoder: a slot loads into an empty sequence");
    FILE* f = std::fopen(path.c_str(), "rb");
    if (f == nullptr) throw KvError("kv8 decoder: cannot open the slot " + path);
    std::vector<uint8_t> host;
    uint8_t buf[1 << 16];
    for (size_t n; (n = std::fread(buf, 1, sizeof buf, f)) > 0;) host.insert(host.end(), buf, buf + n);
    std::fclose(f);
    int32_t np = 0, len = 0;
    if (yahkv_kv8_slot_check(&g_, host.data(), host.size(), &np, &len) != YAHKV_OK)
      throw KvError("kv8 decoder: the slot " + path + " does not match this geometry");
    // the header's page count is the one the tokens need, and the sequence's row holds exactly those pages: a slot
    // never reaches pages the sequence does not own
    if (np != (len + g_.page_tokens - 1) / g_.page_tokens || np > stride_)
      throw KvError("kv8 decoder: the slot " + path + " names more pages than its tokens fill");
    Reserve(seq, len);
    if (int32_t(pages_[size_t(seq)].size()) != np) throw KvError("kv8 decoder: the slot " + path + " does not fit the sequence");
    Upload();
    DeviceBuffer slot(host.size());
    CheckHip(hipMemcpyAsync(slot.get(), host.data(), host.size(), hipMemcpyHostToDevice, stream_), "slot");
    const yahkv_kv8_pools pools = PoolsOf(st_);
    Check(yahkv_kv8_slot_unpack(&g_, &pools, static_cast<const int32_t*>(st_.ptab.ptr) + size_t(seq) * stride_, np,
                                slot.get(), stream_), "kv8_slot_unpack");
    CheckHip(hipStreamSynchronize(stream_), "slot");
    len_[size_t(seq)] = len;
    open_at_[size_t(seq)] = len;
    return len;
  }

  // The next Step of `seq` writes position pos. With quantized V the open tile must hold the keys since the last 16-key
  // boundary: pos is such a boundary, or the position the open tile was last written up to (by a Step, or seeded by the
  // prefill: SeedOpenTile, loom_prefill.hpp:944-947) (loom_decoder.hpp:233-235).
  void ResumeAt(int32_t seq, int32_t pos) {
    if (pos < 0 || pos > T_) throw KvError("kv8 decoder: position past the context");
    if (pos % 16 != 0 && pos != open_at_.at(size_t(seq)))
      throw KvError("kv8 decoder: steps over quantized V must be contiguous from a 16-key boundary");
    Reserve(seq, pos);
    len_.at(size_t(seq)) = pos;
    open_at_[size_t(seq)] = pos;
  }
  // (for the prefill: the chunk append has left the newest tile in the open tile up to `len`)
  void SeedOpenTile(int32_t seq, int32_t len) { len_.at(size_t(seq)) = len, open_at_[size_t(seq)] = len; }

  // One decode step for sequences 0 .. n_seqs - 1: K / V rows [n_seqs][H][256] appended at each sequence's length, then
  // q [n_seqs][n_q][256] attends over the lengthened sequences into out f32. LoomDecoder::Step's kappend, vappend,
  // part_q, reduce (loom_decoder.hpp:253-268) in two dispatches (yahkv_kv8_decode_step).
  void Step(int32_t n_seqs, const void* k, const void* v, int32_t kv_dtype, const void* q, int32_t q_dtype,
            float softmax_scale, const float* gate, float* out) {
    if (!bound_) throw KvError("kv8 decoder: no state bound");
    if (n_seqs <= 0 || n_seqs > max_seqs_) throw KvError("kv8 decoder: bad batch");
    for (int32_t s = 0; s < n_seqs; ++s) {
      if (len_[size_t(s)] >= T_) throw KvError("kv8 decoder: position past the set's context");
      if (len_[size_t(s)] % 16 != 0 && len_[size_t(s)] != open_at_[size_t(s)])
        throw KvError("kv8 decoder: steps over quantized V must be contiguous from a 16-key boundary");
    }
    const size_t slot = step_ % kStaging;
    if (step_ >= kStaging) CheckHip(hipEventSynchronize(staged_[slot]), "lengths");
    int32_t* row = len_host_ + slot * size_t(max_seqs_);
    for (int32_t s = 0; s < max_seqs_; ++s) row[s] = 0;
    for (int32_t s = 0; s < n_seqs; ++s) {
      Reserve(s, len_[size_t(s)] + 1);
      row[s] = ++len_[size_t(s)];
      open_at_[size_t(s)] = len_[size_t(s)];
    }
    Upload();
    CheckHip(hipMemcpyAsync(len_dev_.get(), row, sizeof(int32_t) * size_t(max_seqs_), hipMemcpyHostToDevice, stream_), "lengths");
    CheckHip(hipEventRecord(staged_[slot], stream_), "lengths");
    ++step_;
    const yahkv_kv8_pools pools = PoolsOf(st_);
    Check(yahkv_kv8_decode_step(&g_, &pools, static_cast<const int32_t*>(st_.ptab.ptr), stride_,
                                static_cast<const int32_t*>(len_dev_.get()), n_seqs, T_, k, v, kv_dtype, q, q_dtype,
                                softmax_scale, gate, out, workspace_.get(), workspace_.size(), nullptr, stream_),
          "kv8_decode_step");
  }

  // Validates and uploads the page table if it changed (loom_prefill.hpp:1306-1319).
  void Upload() {
    if (!table_dirty_) return;
    std::vector<int32_t> owned(static_cast<size_t>(max_seqs_), 0);
    for (int32_t s = 0; s < max_seqs_; ++s) owned[size_t(s)] = int32_t(pages_[size_t(s)].size()) * g_.page_tokens;
    // forked sequences share their full pages: a page may appear as often as the allocator has it retained
    Check(yahkv_validate_shared_page_table(&g_, pool_->handle(), table_.data(), stride_, owned.data(), max_seqs_),
          "page table");
    CheckHip(hipMemcpyAsync(st_.ptab.ptr, table_.data(), sizeof(int32_t) * table_.size(), hipMemcpyHostToDevice, stream_),
             "page table upload");
    CheckHip(hipStreamSynchronize(stream_), "page table upload");
    table_dirty_ = false;
  }

 private:
  yahkv_geometry g_;
  int32_t max_seqs_, T_, stride_ = 0;
  hipStream_t stream_;
  std::vector<int32_t> table_, len_, open_at_;
  std::vector<std::vector<int32_t>> pages_;
  std::vector<DeviceBuffer> own_;
  std::unique_ptr<PagePool> pool_;
  DeviceBuffer len_dev_, workspace_;
  static constexpr size_t kStaging = 4;
  int32_t* len_host_ = nullptr;  // [kStaging][max_seqs]
  hipEvent_t staged_[kStaging] = {nullptr, nullptr, nullptr, nullptr};
  size_t step_ = 0;
  Kv8DecoderState st_;
  bool bound_ = false, table_dirty_ = true;
};

// Chunked prefill of one layer on the decoder's state (loom_prefill.hpp:3343-3410): the channel means from a sequence's
// first chunk, the chunk's K and V quantized into newly reserved pages with the newest tile left open, then causal
// attention of the chunk's queries over prefix + chunk.
class Kv8Prefill {
 public:
  explicit Kv8Prefill(Kv8Decoder& dec) : dec_(dec), prefix_dev_(sizeof(int32_t) * 1024) {}

  // Sequences 0 .. n_seqs - 1 each take `chunk_len` more tokens: k / v [n_seqs][chunk_len][H][256] of kv_dtype,
  // q [n_seqs][chunk_len][n_q][256] bf16, out of out_dtype. The sequences must all be at their first chunk or all past
  // it (the means are computed for the whole batch or not at all). Afterwards the decoder continues at the new lengths.
  void RunChunk(int32_t n_seqs, int32_t chunk_len, const void* k, const void* v, int32_t kv_dtype, const void* q,
                float softmax_scale, const float* gate, void* out, int32_t out_dtype) {
    if (n_seqs <= 0 || n_seqs > 1024) throw KvError("kv8 prefill: bad batch");
    std::vector<int32_t> prefix(static_cast<size_t>(n_seqs));
    int32_t max_prefix = 0, first = 0;
    for (int32_t s = 0; s < n_seqs; ++s) {
      prefix[size_t(s)] = dec_.length(s);
      max_prefix = std::max(max_prefix, prefix[size_t(s)]);
      first += prefix[size_t(s)] == 0;
      dec_.Reserve(s, prefix[size_t(s)] + chunk_len);
    }
    if (first != 0 && first != n_seqs) throw KvError("kv8 prefill: first chunks and later chunks in one call");
    dec_.Upload();
    CheckHip(hipMemcpyAsync(prefix_dev_.get(), prefix.data(), sizeof(int32_t) * prefix.size(), hipMemcpyHostToDevice,
                            dec_.stream()), "prefix lengths");
    CheckHip(hipStreamSynchronize(dec_.stream()), "prefix lengths");
    const yahkv_kv8_pools pools = PoolsOf(dec_.state());
    const int32_t* ptab = static_cast<const int32_t*>(dec_.state().ptab.ptr);
    const int32_t* pre = static_cast<const int32_t*>(prefix_dev_.get());
    const int32_t stride = dec_.page_table_stride();
    if (first != 0)  // yah_kmean on chunk 0 only (loom_prefill.hpp:3343-3345)
      Check(yahkv_kv8_kmean(&dec_.geometry(), &pools, ptab, stride, nullptr, n_seqs, chunk_len, k, kv_dtype, dec_.stream()),
            "kv8_kmean");
    Check(yahkv_kv8_append(&dec_.geometry(), &pools, ptab, stride, pre, nullptr, n_seqs, chunk_len, k, v, kv_dtype,
                           dec_.stream()), "kv8_append");
    const size_t need = yahkv_kv8_prefill_workspace_bytes(&dec_.geometry(), n_seqs, max_prefix, chunk_len);
    if (need > images_.size()) {
      CheckHip(hipStreamSynchronize(dec_.stream()), "prefill workspace");
      images_ = DeviceBuffer(need);
    }
    Check(yahkv_kv8_prefill_attend(&dec_.geometry(), &pools, ptab, stride, pre, n_seqs, max_prefix, chunk_len, q,
                                   softmax_scale, gate, out, out_dtype, images_.get(), images_.size(), dec_.stream()),
          "kv8_prefill_attend");
    for (int32_t s = 0; s < n_seqs; ++s) dec_.SeedOpenTile(s, prefix[size_t(s)] + chunk_len);
  }

 private:
  Kv8Decoder& dec_;
  DeviceBuffer prefix_dev_, images_;
};

}  // namespace yahkv_host

#endif  // YAHKV_KV8_CACHE_HPP_
