// Reader for the reference's own slot files ("YAHSLOT1", LoomPrefill::SaveState, engine/model/loom_prefill.hpp:976-1024):
// a header of five u64 {magic, T (context), B (chunk size), chunks, nbufs} followed by ten buffers, each a u64 byte
// count and the raw bytes, in the order of StateBuffers() (:1027-1030): page table, kq, ks, km, vq, vs, the f16 K pool,
// the f16 V^T pool, the convolution rings, the DeltaNet states. The six KV buffers hold every full-attention layer one
// after the other (DecoderState(), :952-972) in the layouts of kv8.hpp, which are the reference's, so a layer's pages
// load into kv8a16 / kv4a16 pools here as plain copies: page by page, from the slot's physical pages (through its page
// table) to any pages of the caller's pool. The recurrent states are not part of this library and are skipped.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <cstring>

#include "kv8.hpp"

namespace {

constexpr uint64_t kRefSlotMagic = 0x31544f4c53484159ull;  // "YAHSLOT1"
enum { kPtab = 0, kKq, kKs, kKm, kVq, kVs, kKpool, kVtpool, kConv, kState, kBuffers };

uint64_t ReadU64(const unsigned char* p) {
  uint64_t v;
  std::memcpy(&v, p, 8);
  return v;
}

}  // namespace

extern "C" int yahkv_refslot_parse(const void* file, size_t file_bytes, yahkv_refslot_info* info) {
  if (file == nullptr || info == nullptr) return YAHKV_ERR_ARG;
  const unsigned char* p = static_cast<const unsigned char*>(file);
  if (file_bytes < 40 || ReadU64(p) != kRefSlotMagic) return YAHKV_ERR_ARG;
  yahkv_refslot_info out{};
  out.context = ReadU64(p + 8), out.chunk = ReadU64(p + 16), out.chunks = ReadU64(p + 24);
  if (ReadU64(p + 32) != kBuffers) return YAHKV_ERR_SHAPE;  // another set of state buffers: not a slot of the paged sets
  size_t at = 40;
  for (int b = 0; b < kBuffers; ++b) {
    if (file_bytes - at < 8) return YAHKV_ERR_ARG;
    const uint64_t n = ReadU64(p + at);
    at += 8;
    if (n > file_bytes - at) return YAHKV_ERR_ARG;  // truncated
    out.offset[b] = at, out.size[b] = n;
    at += n;
  }
  // The page table: one i32 per 256-token page of the pools; the pools' rows are pages * 256 (pool_rows(), :974).
  if (out.size[kPtab] == 0 || out.size[kPtab] % 4 != 0 || out.size[kPtab] / 4 > 0x7fffff) return YAHKV_ERR_SHAPE;
  out.n_pages = static_cast<int32_t>(out.size[kPtab] / 4);
  const uint64_t rows = uint64_t(out.n_pages) * 256;
  // Four kv heads of 256 dims: km is 4096 bytes per layer (:958). Bits from the ratio of codes to scales:
  // kq / ks = 1024 / 32 (8 bits) or 512 / 128 (4 bits) per row; vq / vs = 1024 / 256 or 512 / 256.
  if (out.size[kKm] == 0 || out.size[kKm] % 4096 != 0) return YAHKV_ERR_SHAPE;  // a set with f16 K: no quantized pools to load
  const uint64_t layers = out.size[kKm] / 4096;
  int kb = 0, vb = 0;
  if (out.size[kKq] == layers * rows * 1024 && out.size[kKs] == layers * rows * 32) kb = 8;
  if (out.size[kKq] == layers * rows * 512 && out.size[kKs] == layers * rows * 128) kb = 4;
  if (out.size[kVq] == layers * rows * 1024 && out.size[kVs] == layers * rows * 256) vb = 8;
  if (out.size[kVq] == layers * rows * 512 && out.size[kVs] == layers * rows * 256) vb = 4;
  if (kb == 0 || vb == 0 || layers > 0x7fffffff) return YAHKV_ERR_SHAPE;
  out.n_layers = static_cast<int32_t>(layers), out.n_kv_heads = 4;
  out.format = kb == 8 ? (vb == 8 ? YAHKV_KV8A16 : YAHKV_K8V4A16) : (vb == 4 ? YAHKV_KV4A16 : YAHKV_K4V8A16);
  if (out.chunks * out.chunk > rows) return YAHKV_ERR_SHAPE;
  const int32_t* ptab = reinterpret_cast<const int32_t*>(p + out.offset[kPtab]);
  for (int32_t i = 0; i < out.n_pages; ++i) {  // (unaligned reads: the file is bytes)
    int32_t e;
    std::memcpy(&e, reinterpret_cast<const unsigned char*>(ptab) + 4 * size_t(i), 4);
    if (e < 0 || e >= out.n_pages) return YAHKV_ERR_PAGE;
  }
  *info = out;
  return YAHKV_OK;
}

extern "C" int yahkv_refslot_load_layer(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const void* file,
                                        size_t file_bytes, int32_t layer, const int32_t* pages, int32_t n_pages,
                                        void* stream) {
  yahkv_refslot_info info;
  if (const int rc = yahkv_refslot_parse(file, file_bytes, &info)) return rc;
  if (const int rc = yahkv::CheckKv8Pools(g, pools)) return rc;
  if (g->format != info.format || g->n_kv_heads != info.n_kv_heads) return YAHKV_ERR_SHAPE;
  if (layer < 0 || layer >= info.n_layers || pages == nullptr) return YAHKV_ERR_ARG;
  const uint64_t tokens = info.chunks * info.chunk;
  const int32_t used = static_cast<int32_t>((tokens + 255) / 256);
  if (n_pages < used || n_pages < 1) return YAHKV_ERR_ARG;
  for (int32_t i = 0; i < std::max(used, 1); ++i)
    if (pages[i] < 0 || pages[i] >= g->n_pages) return YAHKV_ERR_PAGE;
  const yahkv::Kv8Geom kg = yahkv::MakeKv8Geom(*g);
  const unsigned char* p = static_cast<const unsigned char*>(file);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const size_t k_row = size_t(kg.n_kv) * kg.kq_head() * 4, s_row = size_t(kg.n_kv) * kg.ks_head() * 4;  // bytes per token
  const size_t v_tile = size_t(256) * kg.vq_dim() * 4, s_tile = size_t(256) * 4;                        // bytes per (head, tile)
  const size_t ref_tiles = size_t(info.n_pages) * 16;
  auto copy = [&](void* dst, const unsigned char* src, size_t n) {
    return hipMemcpyAsync(dst, src, n, hipMemcpyHostToDevice, st) == hipSuccess;
  };
  bool ok = true;
  for (int32_t lp = 0; lp < used && ok; ++lp) {
    int32_t rp;
    std::memcpy(&rp, p + info.offset[kPtab] + 4 * size_t(lp), 4);
    const size_t dp = size_t(pages[lp]);
    ok = ok && copy(static_cast<char*>(pools->kq) + dp * 256 * k_row,
                    p + info.offset[kKq] + (size_t(layer) * info.n_pages + rp) * 256 * k_row, 256 * k_row);
    ok = ok && copy(static_cast<char*>(pools->ks) + dp * 256 * s_row,
                    p + info.offset[kKs] + (size_t(layer) * info.n_pages + rp) * 256 * s_row, 256 * s_row);
    for (int h = 0; h < kg.n_kv && ok; ++h) {  // V^T: [kv head][tile][256 dims][codes], 16 tiles per page
      ok = ok && copy(static_cast<char*>(pools->vq) + (size_t(h) * kg.tiles() + dp * 16) * v_tile,
                      p + info.offset[kVq] + ((size_t(layer) * kg.n_kv + h) * ref_tiles + size_t(rp) * 16) * v_tile, 16 * v_tile);
      ok = ok && copy(static_cast<char*>(pools->vs) + (size_t(h) * kg.tiles() + dp * 16) * s_tile,
                      p + info.offset[kVs] + ((size_t(layer) * kg.n_kv + h) * ref_tiles + size_t(rp) * 16) * s_tile, 16 * s_tile);
    }
  }
  // the layer's channel means go to the sequence's first page here
  ok = ok && copy(static_cast<char*>(pools->km) + size_t(pages[0]) * kg.W() * 4, p + info.offset[kKm] + size_t(layer) * 4096, 4096);
  // A slot ends on a whole chunk, a multiple of 16 tokens: the next key opens a new tile, and the open tile's bytes are
  // not read before they are written (loom_decoder.hpp:233-235).
  if (!ok || hipStreamSynchronize(st) != hipSuccess) return YAHKV_ERR_LAUNCH;  // the file's memory is the caller's again
  return YAHKV_OK;
}
