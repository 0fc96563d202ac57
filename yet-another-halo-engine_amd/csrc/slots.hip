// Whole-page moves: copies between pages of the pools (a forked sequence gets its own copy of the shared prefix's
// last, partly filled page) and slots (the pages of one sequence, in logical order, packed into one buffer and back).
//
// The reference saves a sequence state as `{magic, T, B, chunks, nbufs}` followed by each state buffer, raw, with its
// size in front (engine/model/loom_prefill.hpp:976-1024); its buffers hold one sequence, so it dumps them whole. Here a
// sequence owns pages scattered over shared pools, so a slot holds only that sequence's pages, gathered through its
// page-table row; it loads into any free pages of a pool of the same geometry.
#include "common.hpp"
#include "kv8.hpp"

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

// The same for the reference's own formats (kv8.hpp). A page's share of the six buffers is 4 + 2 H contiguous pieces:
// its 256 rows of kq and of ks, its channel means, its open tile, and per kv head its 16 tiles of vq and of vs (V^T lies
// [kv head][tile]). A slot's body is a set of pools of the slot's own page count with the identity page table, in the
// reference's layouts: kq, ks, km, vq, vs, vopen one after the other.
struct Kv8Piece {
  char* base;       // the pool buffer
  size_t bytes;     // of the piece
  size_t page, head;  // byte strides: from page to page, and from kv head to kv head of a pool of `pages` pages
};
__device__ inline Kv8Piece PieceOf(const Kv8Geom& g, const Kv8Pools& p, int which, size_t pages, size_t* in_slot) {
  const size_t W = size_t(g.W());
  const size_t kq = size_t(256) * g.n_kv * g.kq_head() * 4, ks = size_t(256) * g.n_kv * g.ks_head() * 4, km = W * 4;
  const size_t vq = size_t(16) * 256 * g.vq_dim() * 4, vs = size_t(16) * 256 * 4, vo = W * 16 * 2;
  // where each buffer starts in a slot of `pages` pages
  const size_t o_ks = kq * pages, o_km = o_ks + ks * pages, o_vq = o_km + km * pages;
  const size_t o_vs = o_vq + vq * pages * g.n_kv, o_vo = o_vs + vs * pages * g.n_kv;
  if (which == 0) return *in_slot = 0, Kv8Piece{reinterpret_cast<char*>(p.kq), kq, kq, 0};
  if (which == 1) return *in_slot = o_ks, Kv8Piece{reinterpret_cast<char*>(p.ks), ks, ks, 0};
  if (which == 2) return *in_slot = o_km, Kv8Piece{reinterpret_cast<char*>(p.km), km, km, 0};
  if (which == 3) return *in_slot = o_vo, Kv8Piece{reinterpret_cast<char*>(p.vo), vo, vo, 0};
  const int h = (which - 4) % g.n_kv;
  if (which - 4 < g.n_kv) return *in_slot = o_vq + vq * pages * h, Kv8Piece{reinterpret_cast<char*>(p.vq), vq, vq, vq * g.tiles() / 16 * h};
  return *in_slot = o_vs + vs * pages * h, Kv8Piece{reinterpret_cast<char*>(p.vs), vs, vs, vs * g.tiles() / 16 * h};
}
// grid.x = copies, grid.y = piece; modes as MovePages
__global__ __launch_bounds__(256) void Kv8MovePages(Kv8Geom g, Kv8Pools pools, int32_t format, const int32_t* src,
                                                    const int32_t* dst, int mode, char* slot, int32_t n_pages,
                                                    int32_t n_tokens) {
  const int i = blockIdx.x;
  size_t off_in_slot;
  const Kv8Piece pc = PieceOf(g, pools, blockIdx.y, size_t(n_pages), &off_in_slot);
  char* in_slot = slot == nullptr ? nullptr : slot + kSlotHeaderBytes + off_in_slot + pc.bytes * size_t(i);
  char* pool = pc.base + pc.head;
  const char* from;
  char* to;
  if (mode == 0) {
    from = pool + pc.page * size_t(ClampPage(src[i], g.n_pages)), to = pool + pc.page * size_t(ClampPage(dst[i], g.n_pages));
  } else if (mode == 1) {
    from = pool + pc.page * size_t(ClampPage(src[i], g.n_pages)), to = in_slot;
  } else {
    from = in_slot, to = pool + pc.page * size_t(ClampPage(dst[i], g.n_pages));
  }
  for (size_t o = size_t(threadIdx.x) * 16; o < pc.bytes; o += 256 * 16)
    *reinterpret_cast<uint4*>(to + o) = *reinterpret_cast<const uint4*>(from + o);
  if (mode == 1 && i == 0 && blockIdx.y == 0 && threadIdx.x == 0) {
    uint64_t* h = reinterpret_cast<uint64_t*>(slot);
    h[0] = kSlotMagic, h[1] = uint64_t(format), h[2] = uint64_t(g.n_kv), h[3] = kKv8Dim, h[4] = kKv8Page;
    h[5] = uint64_t(n_pages), h[6] = uint64_t(n_tokens), h[7] = 6;
  }
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" int yahkv_kv8_copy_pages(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* src_pages,
                                    const int32_t* dst_pages, int32_t n, void* stream) {
  if (const int st = CheckKv8Pools(g, pools)) return st;
  if (n < 0 || (n > 0 && (src_pages == nullptr || dst_pages == nullptr))) return YAHKV_ERR_ARG;
  if (n == 0) return YAHKV_OK;
  hipLaunchKernelGGL(Kv8MovePages, dim3(static_cast<unsigned>(n), static_cast<unsigned>(4 + 2 * g->n_kv_heads)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), MakeKv8Geom(*g), MakeKv8Pools(*pools), g->format, src_pages,
                     dst_pages, 0, nullptr, n, 0);
  return LaunchStatus();
}

extern "C" size_t yahkv_kv8_slot_bytes(const yahkv_geometry* g, int32_t n_pages) {
  if (CheckKv8Geometry(g) || n_pages <= 0) return 0;
  yahkv_geometry one = *g;
  one.n_pages = 1;  // a page's share of every buffer
  const size_t per_page = yahkv_kv8_kq_bytes(&one) + yahkv_kv8_ks_bytes(&one) + yahkv_kv8_km_bytes(&one) +
                          yahkv_kv8_vq_bytes(&one) + yahkv_kv8_vs_bytes(&one) + yahkv_kv8_vopen_bytes(&one);
  return kSlotHeaderBytes + per_page * size_t(n_pages);
}

extern "C" int yahkv_kv8_slot_pack(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* table_row,
                                   int32_t n_pages, int32_t n_tokens, void* slot, void* stream) {
  if (const int st = CheckKv8Pools(g, pools)) return st;
  if (table_row == nullptr || slot == nullptr || n_pages <= 0 || n_tokens < 0) return YAHKV_ERR_ARG;
  if (int64_t(n_tokens) > int64_t(n_pages) * kKv8Page || (reinterpret_cast<uintptr_t>(slot) & 15)) return YAHKV_ERR_ARG;
  hipLaunchKernelGGL(Kv8MovePages, dim3(static_cast<unsigned>(n_pages), static_cast<unsigned>(4 + 2 * g->n_kv_heads)),
                     dim3(256), 0, static_cast<hipStream_t>(stream), MakeKv8Geom(*g), MakeKv8Pools(*pools), g->format,
                     table_row, nullptr, 1, static_cast<char*>(slot), n_pages, n_tokens);
  return LaunchStatus();
}

extern "C" int yahkv_kv8_slot_check(const yahkv_geometry* g, const void* header, size_t slot_bytes, int32_t* n_pages,
                                    int32_t* n_tokens) {
  if (const int st = CheckKv8Geometry(g)) return st;
  if (header == nullptr || slot_bytes < size_t(kSlotHeaderBytes)) return YAHKV_ERR_ARG;
  const uint64_t* h = static_cast<const uint64_t*>(header);
  if (h[0] != kSlotMagic || h[7] != 6) return YAHKV_ERR_ARG;
  if (h[1] != uint64_t(g->format) || h[2] != uint64_t(g->n_kv_heads) || h[3] != uint64_t(kKv8Dim) || h[4] != uint64_t(kKv8Page))
    return YAHKV_ERR_SHAPE;
  if (h[5] == 0 || h[5] > 0x7FFFFFFFu || h[6] == 0 || h[5] != (h[6] + h[4] - 1) / h[4]) return YAHKV_ERR_ARG;
  if (yahkv_kv8_slot_bytes(g, static_cast<int32_t>(h[5])) != slot_bytes) return YAHKV_ERR_ARG;
  if (n_pages != nullptr) *n_pages = static_cast<int32_t>(h[5]);
  if (n_tokens != nullptr) *n_tokens = static_cast<int32_t>(h[6]);
  return YAHKV_OK;
}

extern "C" int yahkv_kv8_slot_unpack(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* table_row,
                                     int32_t n_pages, const void* slot, void* stream) {
  if (const int st = CheckKv8Pools(g, pools)) return st;
  if (table_row == nullptr || slot == nullptr || n_pages <= 0 || (reinterpret_cast<uintptr_t>(slot) & 15))
    return YAHKV_ERR_ARG;
  hipLaunchKernelGGL(Kv8MovePages, dim3(static_cast<unsigned>(n_pages), static_cast<unsigned>(4 + 2 * g->n_kv_heads)),
                     dim3(256), 0, static_cast<hipStream_t>(stream), MakeKv8Geom(*g), MakeKv8Pools(*pools), g->format,
                     nullptr, table_row, 2, static_cast<char*>(const_cast<void*>(slot)), n_pages, 0);
  return LaunchStatus();
}

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
