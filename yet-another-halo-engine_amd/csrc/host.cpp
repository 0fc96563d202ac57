// Host-only entry points of include/yahkv.h: geometry checks, pool sizes, page-table validation and the page allocator.
#include <algorithm>
#include <cstdint>
#include <functional>
#include <new>
#include <vector>

#include "common.hpp"
#include "kv8.hpp"

namespace yahkv {

int CheckGeometry(const yahkv_geometry* g) {
  if (g == nullptr) return YAHKV_ERR_ARG;
  if (g->format != YAHKV_Q8_0 && g->format != YAHKV_Q4_0) return YAHKV_ERR_SHAPE;
  if (g->n_q_heads <= 0 || g->n_kv_heads <= 0 || g->n_pages <= 0) return YAHKV_ERR_ARG;
  if (g->n_q_heads % g->n_kv_heads != 0 || g->n_q_heads / g->n_kv_heads > 8) return YAHKV_ERR_SHAPE;
  if (g->head_dim != 128 && g->head_dim != 256) return YAHKV_ERR_SHAPE;
  if (g->page_tokens != 16 && g->page_tokens != 32 && g->page_tokens != 64) return YAHKV_ERR_SHAPE;
  return YAHKV_OK;
}

int CheckPools(const yahkv_geometry* g, const yahkv_pools* pools) {
  if (const int st = CheckGeometry(g)) return st;
  if (pools == nullptr || pools->kq == nullptr || pools->ks == nullptr || pools->vq == nullptr || pools->vs == nullptr)
    return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(pools->kq) | reinterpret_cast<uintptr_t>(pools->ks) |
       reinterpret_cast<uintptr_t>(pools->vq) | reinterpret_cast<uintptr_t>(pools->vs)) & 15)
    return YAHKV_ERR_ARG;
  // the kernels address pages 0 .. n_pages - 1 of every pool: a shorter buffer is refused here, before any launch
  if (pools->kq_bytes < yahkv_kq_bytes(g) || pools->ks_bytes < yahkv_ks_bytes(g) ||
      pools->vq_bytes < yahkv_vq_bytes(g) || pools->vs_bytes < yahkv_vs_bytes(g))
    return YAHKV_ERR_ARG;
  return YAHKV_OK;
}

}  // namespace yahkv

using yahkv::CheckGeometry;
using yahkv::MakeGeom;

extern "C" {

const char* yahkv_version(void) { return "yahkv 0.1 (gfx950)"; }

const char* yahkv_strerror(int status) {
  switch (status) {
    case YAHKV_OK: return "ok";
    case YAHKV_ERR_ARG: return "bad argument (null or misaligned pointer, non-positive count, pool shorter than the geometry needs)";
    case YAHKV_ERR_SHAPE: return "no kernel for this geometry";
    case YAHKV_ERR_PAGE: return "page table entry out of range or page used twice";
    case YAHKV_ERR_WORKSPACE: return "workspace too small";
    case YAHKV_ERR_NOMEM: return "page pool exhausted";
    case YAHKV_ERR_LAUNCH: return "kernel launch failed";
    default: return "unknown status";
  }
}

int yahkv_check_geometry(const yahkv_geometry* g) { return CheckGeometry(g); }

size_t yahkv_kq_bytes(const yahkv_geometry* g) {
  return CheckGeometry(g) ? 0 : size_t(g->n_pages) * MakeGeom(*g).code_page();
}
size_t yahkv_ks_bytes(const yahkv_geometry* g) {
  return CheckGeometry(g) ? 0 : size_t(g->n_pages) * MakeGeom(*g).scale_page() * 2;
}
size_t yahkv_vq_bytes(const yahkv_geometry* g) { return yahkv_kq_bytes(g); }
size_t yahkv_vs_bytes(const yahkv_geometry* g) { return yahkv_ks_bytes(g); }

size_t yahkv_bytes_per_token(const yahkv_geometry* g) {
  if (CheckGeometry(g)) return 0;
  const yahkv::Geom m = MakeGeom(*g);
  return size_t(2) * m.n_kv * m.nb() * (m.code_bytes() + 2);
}

namespace {
// owners == nullptr: a page may appear once in the whole table; else page p may appear at most owners[p] times, and
// never twice in one row.
int ValidateTable(const yahkv_geometry* g, const int32_t* table, int32_t page_table_stride, const int32_t* seq_len,
                  int32_t n_seqs, const std::vector<int32_t>* owners) {
  // (the reference's own format has its own geometry check: 256-token pages)
  if (const int st = g != nullptr && yahkv::Kv8BitsK(g->format) != 0 ? yahkv::CheckKv8Geometry(g) : yahkv::CheckGeometry(g)) return st;
  if (table == nullptr || seq_len == nullptr || n_seqs <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  std::vector<int32_t> used(static_cast<size_t>(g->n_pages), 0), row_of(static_cast<size_t>(g->n_pages), -1);
  for (int32_t s = 0; s < n_seqs; ++s) {
    if (seq_len[s] < 0) return YAHKV_ERR_ARG;
    const int64_t np = (int64_t(seq_len[s]) + g->page_tokens - 1) / g->page_tokens;
    if (np > page_table_stride) return YAHKV_ERR_PAGE;
    for (int64_t p = 0; p < np; ++p) {
      const int32_t pg = table[int64_t(s) * page_table_stride + p];
      if (pg < 0 || pg >= g->n_pages) return YAHKV_ERR_PAGE;
      const size_t i = static_cast<size_t>(pg);
      const int32_t limit = owners == nullptr ? 1 : (*owners)[i];
      if (++used[i] > limit || row_of[i] == s) return YAHKV_ERR_PAGE;
      row_of[i] = s;
    }
  }
  return YAHKV_OK;
}
}  // namespace

int yahkv_validate_page_table(const yahkv_geometry* g, const int32_t* table, int32_t page_table_stride,
                              const int32_t* seq_len, int32_t n_seqs) {
  return ValidateTable(g, table, page_table_stride, seq_len, n_seqs, nullptr);
}

// ---- page allocator -------------------------------------------------------------------------------------------

struct yahkv_pagepool {
  std::vector<int32_t> free_list;  // handed out from the back
  std::vector<int32_t> refs;       // owners of a page; 0 = free
};

yahkv_pagepool* yahkv_pagepool_create(int32_t n_pages) {
  if (n_pages <= 0) return nullptr;
  auto* p = new (std::nothrow) yahkv_pagepool;
  if (p == nullptr) return nullptr;
  p->free_list.resize(static_cast<size_t>(n_pages));
  for (int32_t i = 0; i < n_pages; ++i) p->free_list[static_cast<size_t>(i)] = n_pages - 1 - i;  // lowest id first
  p->refs.assign(static_cast<size_t>(n_pages), 0);
  return p;
}

void yahkv_pagepool_destroy(yahkv_pagepool* p) { delete p; }

int32_t yahkv_pagepool_free_count(const yahkv_pagepool* p) {
  return p == nullptr ? 0 : static_cast<int32_t>(p->free_list.size());
}

int yahkv_pagepool_alloc(yahkv_pagepool* p, int32_t n, int32_t* out) {
  if (p == nullptr || n < 0 || (n > 0 && out == nullptr)) return YAHKV_ERR_ARG;
  if (static_cast<size_t>(n) > p->free_list.size()) return YAHKV_ERR_NOMEM;
  for (int32_t i = 0; i < n; ++i) {
    out[i] = p->free_list.back();
    p->free_list.pop_back();
    p->refs[static_cast<size_t>(out[i])] = 1;
  }
  return YAHKV_OK;
}

// One owner less for each page; a page goes back to the free list when its last owner lets go.
int yahkv_pagepool_free(yahkv_pagepool* p, const int32_t* pages, int32_t n) {
  if (p == nullptr || n < 0 || (n > 0 && pages == nullptr)) return YAHKV_ERR_ARG;
  const int32_t total = static_cast<int32_t>(p->refs.size());
  for (int32_t i = 0; i < n; ++i) {  // check everything first: free none on error
    if (pages[i] < 0 || pages[i] >= total || p->refs[static_cast<size_t>(pages[i])] <= 0) return YAHKV_ERR_PAGE;
    for (int32_t j = 0; j < i; ++j)
      if (pages[j] == pages[i]) return YAHKV_ERR_PAGE;
  }
  bool any = false;
  for (int32_t i = 0; i < n; ++i) {
    if (--p->refs[static_cast<size_t>(pages[i])] == 0) {
      p->free_list.push_back(pages[i]);
      any = true;
    }
  }
  // keep "lowest id first": the back of the list is the smallest free id
  if (any) std::sort(p->free_list.begin(), p->free_list.end(), std::greater<int32_t>());
  return YAHKV_OK;
}

// One owner more for each page (a sequence forked from a shared prefix keeps the prefix's full pages).
int yahkv_pagepool_retain(yahkv_pagepool* p, const int32_t* pages, int32_t n) {
  if (p == nullptr || n < 0 || (n > 0 && pages == nullptr)) return YAHKV_ERR_ARG;
  const int32_t total = static_cast<int32_t>(p->refs.size());
  for (int32_t i = 0; i < n; ++i)
    if (pages[i] < 0 || pages[i] >= total || p->refs[static_cast<size_t>(pages[i])] <= 0) return YAHKV_ERR_PAGE;
  for (int32_t i = 0; i < n; ++i) ++p->refs[static_cast<size_t>(pages[i])];
  return YAHKV_OK;
}

int yahkv_validate_shared_page_table(const yahkv_geometry* g, const yahkv_pagepool* p, const int32_t* table,
                                     int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs) {
  if (p == nullptr || g == nullptr || static_cast<int64_t>(p->refs.size()) != g->n_pages) return YAHKV_ERR_ARG;
  return ValidateTable(g, table, page_table_stride, seq_len, n_seqs, &p->refs);
}

int32_t yahkv_pagepool_refcount(const yahkv_pagepool* p, int32_t page) {
  if (p == nullptr || page < 0 || page >= static_cast<int32_t>(p->refs.size())) return -1;
  return p->refs[static_cast<size_t>(page)];
}

void yahkv_pagepool_shuffle(yahkv_pagepool* p, uint64_t seed) {
  if (p == nullptr) return;
  uint64_t x = seed ? seed : 0x9E3779B97F4A7C15ull;  // xorshift64*
  auto next = [&x]() {
    x ^= x >> 12, x ^= x << 25, x ^= x >> 27;
    return x * 0x2545F4914F6CDD1Dull;
  };
  for (size_t i = p->free_list.size(); i > 1; --i) std::swap(p->free_list[i - 1], p->free_list[next() % i]);
}

}  // extern "C"
