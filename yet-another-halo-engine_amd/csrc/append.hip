// Token append: block-quantize K and V rows and scatter them into their pages; and the inverse gather used by tests.
//
// Arithmetic is the reference's QuantizeQ8_0 (engine/core/gguf_quant.cpp:310-320), bit for bit: amax over the 32
// elements, d = amax / 127 (IEEE division), inv = d > 0 ? 1 / d : 0, code = lround(x * inv) (halves away from zero),
// stored scale = f16(d) (round to nearest even). q4_0 follows ggml's quantize_row_q4_0_ref.
// Placement follows the reference's page mapping (engine/gpu/loom/tools/gen_kvq.py:48-71): token at position p goes
// to page table[p / PT] (clamped into the pool), slot p % PT.
#include "common.hpp"
#include "quant.hpp"

namespace yahkv {
namespace {

struct AppendArgs {
  Geom g;
  Pools pools;
  const int32_t* table;
  int32_t stride;
  const int32_t* start_pos;
  const int32_t* n_valid;
  int32_t n_seqs, n_new;
  const void* k_src;
  const void* v_src;
  int32_t src_dtype;
};

// One thread per (K|V, sequence, new token, kv head, block): 64 work items per token at 4 kv heads x 256 dims.
// The K block is stored as two 16-byte writes; the V block's bytes go to 32 rows of the transposed page.
template <int FMT>
__global__ __launch_bounds__(256) void AppendBlocks(const AppendArgs a) {
  const Geom g = a.g;
  const int NB = g.nb(), H = g.n_kv, PT = g.pt, D = g.hd;
  const int64_t per_side = int64_t(a.n_seqs) * a.n_new * H * NB;
  const int64_t idx = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= 2 * per_side) return;
  const bool is_v = idx >= per_side;
  int64_t r = is_v ? idx - per_side : idx;
  const int b = int(r % NB);
  r /= NB;
  const int h = int(r % H);
  r /= H;
  const int i = int(r % a.n_new);
  const int s = int(r / a.n_new);
  if (a.n_valid != nullptr && i >= a.n_valid[s]) return;  // padding row of a short chunk

  int pos = a.start_pos[s] + i;
  pos = min(max(pos, 0), a.stride * PT - 1);  // gen_decode_attn.py:59-63
  const int page = ClampPage(a.table[int64_t(s) * a.stride + pos / PT], g.n_pages);
  const int t = pos % PT;

  const void* src = is_v ? a.v_src : a.k_src;
  const size_t off = ((size_t(s) * a.n_new + i) * H + h) * D + size_t(b) * 32;
  float x[32];
#pragma unroll
  for (int j = 0; j < 32; ++j) x[j] = LoadSrc(src, off + j, a.src_dtype);

  alignas(16) uint8_t code[32];
  uint16_t hd;
  QuantizeBlock<FMT>(x, code, &hd);
  StoreBlock<FMT>(g, a.pools, is_v, page, t, h, b, code, hd);
}

// One thread per (K|V, token, kv head, block): the block back in ggml order (scale, then codes).
template <int FMT>
__global__ __launch_bounds__(256) void GatherBlocks(Geom g, Pools pools, const int32_t* table_row, int n_tokens,
                                                     uint8_t* dst_k, uint8_t* dst_v) {
  const int NB = g.nb(), H = g.n_kv, PT = g.pt;
  constexpr int CB = FMT == 8 ? 32 : 16;
  const int64_t per_side = int64_t(n_tokens) * H * NB;
  const int64_t idx = int64_t(blockIdx.x) * blockDim.x + threadIdx.x;
  if (idx >= 2 * per_side) return;
  const bool is_v = idx >= per_side;
  int64_t r = is_v ? idx - per_side : idx;
  const int b = int(r % NB);
  r /= NB;
  const int h = int(r % H);
  const int p = int(r / H);
  const int page = ClampPage(table_row[p / PT], g.n_pages);
  const int t = p % PT;
  const size_t ph = size_t(page) * H + h;
  uint8_t* out = (is_v ? dst_v : dst_k) + ((size_t(p) * H + h) * NB + b) * (CB + 2);
  uint16_t hd;
  if (!is_v) {
    hd = pools.ks[(ph * PT + t) * NB + b];
    const uint8_t* src = pools.kq + ((ph * NB + b) * PT + t) * CB;
    for (int j = 0; j < CB; ++j) out[2 + j] = src[j];
  } else {
    hd = pools.vs[(ph * NB + b) * PT + t];
    const uint8_t* src = pools.vq + (ph * NB + b) * CB * PT + t;
    for (int j = 0; j < CB; ++j) out[2 + j] = src[size_t(j) * PT];
  }
  out[0] = static_cast<uint8_t>(hd & 0xFF);
  out[1] = static_cast<uint8_t>(hd >> 8);
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" int yahkv_append(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                            int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid,
                            int32_t n_seqs, int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype,
                            void* stream) {
  if (const int st = CheckGeometry(g)) return st;
  if (pools == nullptr || pools->kq == nullptr || pools->ks == nullptr || pools->vq == nullptr ||
      pools->vs == nullptr || page_table == nullptr || start_pos == nullptr || k_src == nullptr || v_src == nullptr)
    return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || n_new <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (src_dtype != YAHKV_F32 && src_dtype != YAHKV_F16 && src_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(pools->kq) | reinterpret_cast<uintptr_t>(pools->vq)) & 15) return YAHKV_ERR_ARG;
  AppendArgs a{MakeGeom(*g), MakePools(*pools), page_table, page_table_stride, start_pos, n_valid,
               n_seqs,       n_new,             k_src,      v_src,             src_dtype};
  const int64_t items = int64_t(2) * n_seqs * n_new * a.g.n_kv * a.g.nb();
  const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (g->format == YAHKV_Q8_0)
    hipLaunchKernelGGL(AppendBlocks<8>, dim3(blocks), dim3(256), 0, st, a);
  else
    hipLaunchKernelGGL(AppendBlocks<4>, dim3(blocks), dim3(256), 0, st, a);
  return LaunchStatus();
}

extern "C" int yahkv_gather_blocks(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row,
                                   int32_t n_tokens, void* dst_k, void* dst_v, void* stream) {
  if (const int st = CheckGeometry(g)) return st;
  if (pools == nullptr || table_row == nullptr || dst_k == nullptr || dst_v == nullptr || n_tokens <= 0)
    return YAHKV_ERR_ARG;
  const Geom m = MakeGeom(*g);
  const int64_t items = int64_t(2) * n_tokens * m.n_kv * m.nb();
  const unsigned blocks = static_cast<unsigned>((items + 255) / 256);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (g->format == YAHKV_Q8_0)
    hipLaunchKernelGGL(GatherBlocks<8>, dim3(blocks), dim3(256), 0, st, m, MakePools(*pools), table_row, n_tokens,
                       static_cast<uint8_t*>(dst_k), static_cast<uint8_t*>(dst_v));
  else
    hipLaunchKernelGGL(GatherBlocks<4>, dim3(blocks), dim3(256), 0, st, m, MakePools(*pools), table_row, n_tokens,
                       static_cast<uint8_t*>(dst_k), static_cast<uint8_t*>(dst_v));
  return LaunchStatus();
}
