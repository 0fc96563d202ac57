// Whole-page moves: copies between pages of the pools (a forked sequence gets its own copy of the shared prefix's
// last, partly filled page) and slots (the pages of one sequence, in logical order, packed into one buffer and back).
//
// The reference saves a sequence state as `{magic, T, B, chunks, nbufs}` followed by each state buffer, raw, with its
// size in front (engine/model/loom_prefill.hpp:976-1024); its buffers hold one sequence, so it dumps them whole. Here a
// sequence owns pages scattered over shared pools, so a slot holds only that sequence's pages, gathered through its
// page-table row; it loads into any free pages of a pool of the same geometry.
#include "common.hpp"

namespace yahkv {
namespace {

constexpr uint64_t kSlotMagic = 0x31544F4C53564B59ull;  // "YKVSLOT1"
constexpr int kSlotHeaderBytes = 64;                     // eight u64: magic, format, H, D, PT, pages, tokens, nbufs

struct PageBytes {  // bytes of one page in each pool
  size_t kq, ks, vq, vs;
};
__host__ __device__ inline PageBytes BytesPerPage(const Geom& g) {
  const size_t codes = size_t(g.n_kv) * g.hd * g.pt * (g.format == 8 ? 2 : 1) / 2;
  const size_t scales = size_t(g.n_kv) * g.pt * g.nb() * 2;
  return PageBytes{codes, scales, codes, scales};
}

// grid.x = copies, grid.y = pool (kq, ks, vq, vs); 16 bytes per thread and step. mode 0: page src[i] -> page dst[i] of
// the same pools; 1: page row[i] -> slot; 2: slot -> page row[i].
__global__ __launch_bounds__(256) void MovePages(Geom g, Pools pools, const int32_t* src, const int32_t* dst, int mode,
                                                 char* slot, int32_t n_pages, int32_t n_tokens) {
  const PageBytes pb = BytesPerPage(g);
  const int i = blockIdx.x, which = blockIdx.y;
  const size_t bytes = which == 0 ? pb.kq : which == 1 ? pb.ks : which == 2 ? pb.vq : pb.vs;
  char* base = which == 0   ? reinterpret_cast<char*>(pools.kq)
               : which == 1 ? reinterpret_cast<char*>(pools.ks)
               : which == 2 ? reinterpret_cast<char*>(pools.vq)
                            : reinterpret_cast<char*>(pools.vs);
  // offset of this pool's pages inside a slot
  const size_t before = which == 0 ? 0 : which == 1 ? pb.kq : which == 2 ? pb.kq + pb.ks : pb.kq + pb.ks + pb.vq;
  char* in_slot = slot == nullptr ? nullptr : slot + kSlotHeaderBytes + before * size_t(n_pages) + bytes * size_t(i);
  const char* from;
  char* to;
  if (mode == 0) {
    from = base + bytes * size_t(ClampPage(src[i], g.n_pages)), to = base + bytes * size_t(ClampPage(dst[i], g.n_pages));
  } else if (mode == 1) {
    from = base + bytes * size_t(ClampPage(src[i], g.n_pages)), to = in_slot;
  } else {
    from = in_slot, to = base + bytes * size_t(ClampPage(dst[i], g.n_pages));
  }
  for (size_t o = size_t(threadIdx.x) * 16; o < bytes; o += 256 * 16)
    *reinterpret_cast<uint4*>(to + o) = StreamLoad(reinterpret_cast<const uint4*>(from + o));  // read once
  if (mode == 1 && i == 0 && which == 0 && threadIdx.x == 0) {
    uint64_t* h = reinterpret_cast<uint64_t*>(slot);
    h[0] = kSlotMagic, h[1] = uint64_t(g.format), h[2] = uint64_t(g.n_kv), h[3] = uint64_t(g.hd);
    h[4] = uint64_t(g.pt), h[5] = uint64_t(n_pages), h[6] = uint64_t(n_tokens), h[7] = 4;
  }
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" int yahkv_copy_pages(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* src_pages,
                                const int32_t* dst_pages, int32_t n, void* stream) {
  if (const int st = CheckPools(g, pools)) return st;
  if (n < 0 || (n > 0 && (src_pages == nullptr || dst_pages == nullptr))) return YAHKV_ERR_ARG;
  if (n == 0) return YAHKV_OK;
  hipLaunchKernelGGL(MovePages, dim3(static_cast<unsigned>(n), 4), dim3(256), 0, static_cast<hipStream_t>(stream),
                     MakeGeom(*g), MakePools(*pools), src_pages, dst_pages, 0, nullptr, n, 0);
  return LaunchStatus();
}

extern "C" size_t yahkv_slot_bytes(const yahkv_geometry* g, int32_t n_pages) {
  if (CheckGeometry(g) || n_pages <= 0) return 0;
  const PageBytes pb = BytesPerPage(MakeGeom(*g));
  return kSlotHeaderBytes + (pb.kq + pb.ks + pb.vq + pb.vs) * size_t(n_pages);
}

extern "C" int yahkv_slot_pack(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row,
                               int32_t n_pages, int32_t n_tokens, void* slot, void* stream) {
  if (const int st = CheckPools(g, pools)) return st;
  if (table_row == nullptr || slot == nullptr || n_pages <= 0 || n_tokens < 0) return YAHKV_ERR_ARG;
  if (int64_t(n_tokens) > int64_t(n_pages) * g->page_tokens || (reinterpret_cast<uintptr_t>(slot) & 15))
    return YAHKV_ERR_ARG;
  hipLaunchKernelGGL(MovePages, dim3(static_cast<unsigned>(n_pages), 4), dim3(256), 0,
                     static_cast<hipStream_t>(stream), MakeGeom(*g), MakePools(*pools), table_row, nullptr, 1,
                     static_cast<char*>(slot), n_pages, n_tokens);
  return LaunchStatus();
}

extern "C" int yahkv_slot_check(const yahkv_geometry* g, const void* header, size_t slot_bytes, int32_t* n_pages,
                                int32_t* n_tokens) {
  if (const int st = CheckGeometry(g)) return st;
  if (header == nullptr || slot_bytes < size_t(kSlotHeaderBytes)) return YAHKV_ERR_ARG;
  const uint64_t* h = static_cast<const uint64_t*>(header);
  if (h[0] != kSlotMagic || h[7] != 4) return YAHKV_ERR_ARG;
  if (h[1] != uint64_t(g->format) || h[2] != uint64_t(g->n_kv_heads) || h[3] != uint64_t(g->head_dim) ||
      h[4] != uint64_t(g->page_tokens))
    return YAHKV_ERR_SHAPE;  // a slot loads only into pools of the same format and geometry
  // at least one token, and exactly the pages those tokens fill (a loader trusts the page count for its scatter)
  if (h[5] == 0 || h[5] > 0x7FFFFFFFu || h[6] == 0 || h[5] != (h[6] + h[4] - 1) / h[4]) return YAHKV_ERR_ARG;
  if (yahkv_slot_bytes(g, static_cast<int32_t>(h[5])) != slot_bytes) return YAHKV_ERR_ARG;
  if (n_pages != nullptr) *n_pages = static_cast<int32_t>(h[5]);
  if (n_tokens != nullptr) *n_tokens = static_cast<int32_t>(h[6]);
  return YAHKV_OK;
}

extern "C" int yahkv_slot_unpack(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row,
                                 int32_t n_pages, const void* slot, void* stream) {
  if (const int st = CheckPools(g, pools)) return st;
  if (table_row == nullptr || slot == nullptr || n_pages <= 0 || (reinterpret_cast<uintptr_t>(slot) & 15))
    return YAHKV_ERR_ARG;
  hipLaunchKernelGGL(MovePages, dim3(static_cast<unsigned>(n_pages), 4), dim3(256), 0,
                     static_cast<hipStream_t>(stream), MakeGeom(*g), MakePools(*pools), nullptr, table_row, 2,
                     static_cast<char*>(const_cast<void*>(slot)), n_pages, 0);
  return LaunchStatus();
}
