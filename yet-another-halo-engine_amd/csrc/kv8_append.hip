// kv8a16 (the reference's own KV format, see kv8.hpp): buffer sizes, the channel means, and the two appends: the
// decoder's one token (yah_dattn_kappend + yah_dattn_vappend, gen_decode_attn.py:1043-1107, 436-573) and the prefill's
// chunk (yah_kq8 + yah_vq8 + yah_vseed, gen_kvq.py:166-285, 474-730). Bandwidth-trivial kernels: every load and store
// of a wave is contiguous, and the arithmetic is the reference's, operation for operation (no fused multiply-adds).
#include "kv8.hpp"
#include "quant.hpp"

namespace yahkv {

int CheckKv8Geometry(const yahkv_geometry* g) {
  if (g == nullptr) return YAHKV_ERR_ARG;
  if (Kv8BitsK(g->format) == 0) return YAHKV_ERR_SHAPE;
  if (g->n_q_heads <= 0 || g->n_kv_heads <= 0 || g->n_pages <= 0) return YAHKV_ERR_ARG;
  if (g->n_q_heads % g->n_kv_heads != 0 || g->n_q_heads / g->n_kv_heads > 8) return YAHKV_ERR_SHAPE;
  if (g->head_dim != kKv8Dim || g->page_tokens != kKv8Page) return YAHKV_ERR_SHAPE;
  if (int64_t(g->n_pages) * kKv8Page * g->n_kv_heads * kKv8Dim >= (int64_t(1) << 40)) return YAHKV_ERR_SHAPE;
  return YAHKV_OK;
}

int CheckKv8Pools(const yahkv_geometry* g, const yahkv_kv8_pools* p) {
  if (const int st = CheckKv8Geometry(g)) return st;
  if (p == nullptr || p->kq == nullptr || p->ks == nullptr || p->km == nullptr || p->vq == nullptr || p->vs == nullptr ||
      p->vopen == nullptr)
    return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(p->kq) | reinterpret_cast<uintptr_t>(p->ks) | reinterpret_cast<uintptr_t>(p->km) |
       reinterpret_cast<uintptr_t>(p->vq) | reinterpret_cast<uintptr_t>(p->vs) | reinterpret_cast<uintptr_t>(p->vopen)) & 15)
    return YAHKV_ERR_ARG;
  if (p->kq_bytes < yahkv_kv8_kq_bytes(g) || p->ks_bytes < yahkv_kv8_ks_bytes(g) || p->km_bytes < yahkv_kv8_km_bytes(g) ||
      p->vq_bytes < yahkv_kv8_vq_bytes(g) || p->vs_bytes < yahkv_kv8_vs_bytes(g) ||
      p->vopen_bytes < yahkv_kv8_vopen_bytes(g))
    return YAHKV_ERR_ARG;
  return YAHKV_OK;
}

namespace {

struct Kv8AppendArgs {
  Kv8Geom g;
  Kv8Pools p;
  const int32_t* table;
  int32_t stride;
  const int32_t* start_pos;
  const int32_t* n_valid;
  int32_t n_new;
  const void* k_src;
  const void* v_src;
  int32_t dtype;
};

// first position and number of real tokens of sequence s that lie inside the table; count 0: nothing to write
__device__ __forceinline__ int RealTokens(const Kv8AppendArgs& a, int s, int* p0) {
  const int start = a.start_pos[s];
  int nv = a.n_valid != nullptr ? min(a.n_valid[s], a.n_new) : a.n_new;
  *p0 = start;
  if (start < 0) return 0;
  const long long cap = static_cast<long long>(a.stride) * kKv8Page;
  if (start + static_cast<long long>(nv) > cap) nv = static_cast<int>(max(cap - start, 0ll));
  return max(nv, 0);
}
__device__ __forceinline__ int PageOf(const Kv8AppendArgs& a, int s, int pos) {
  return ClampPage(a.table[int64_t(s) * a.stride + pos / kKv8Page], a.g.n_pages);
}

// One K row of one kv head across a wave, four consecutive dims per lane: centre, scale per 128-dim half (32 lanes),
// codes, stores. `x`: the lane's four source values.
__device__ __forceinline__ void Kv8StoreRowK(const Kv8Geom& g, const Kv8Pools& p, int page0, size_t row, int h, int lane,
                                             float4 x) {
#pragma clang fp contract(off)
  const float4 m = *reinterpret_cast<const float4*>(p.km + g.km_head(page0, h) + 4 * lane);
  const float4 c = {TruncF16(x.x) - m.x, TruncF16(x.y) - m.y, TruncF16(x.z) - m.z, TruncF16(x.w) - m.w};
  float amax = fmaxf(fmaxf(fabsf(c.x), fabsf(c.y)), fmaxf(fabsf(c.z), fabsf(c.w)));
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) amax = fmaxf(amax, __shfl_xor(amax, o, 64));  // over the half's 32 lanes
  float inv;
  uint32_t pair;
  Kv8ScaleK(amax, &inv, &pair);
  p.kq[g.kq_row(row, h) + lane] = Kv8CodesK(c, inv);
  if (lane % 32 == 0) p.ks[g.ks_row(row, h) + lane / 32] = pair;
}
// the same for 4-bit K: rotated, 16 levels per 32-dim group (eight lanes), two lanes per dword
__device__ __forceinline__ void Kv4StoreRowK(const Kv8Geom& g, const Kv8Pools& p, int page0, size_t row, int h, int lane,
                                             float4 x) {
#pragma clang fp contract(off)
  const float4 m = *reinterpret_cast<const float4*>(p.km + g.km_head(page0, h) + 4 * lane);
  const float4 c = {TruncF16(x.x) - m.x, TruncF16(x.y) - m.y, TruncF16(x.z) - m.z, TruncF16(x.w) - m.w};
  uint32_t pair;
  float4 deq;
  uint32_t w = Kv4CodesK(c, lane, &pair, &deq);
  w |= __shfl_xor(w, 1, 64);
  if (lane % 2 == 0) p.kq[g.kq_row(row, h) + lane / 2] = w;
  if (lane % 8 == 0) p.ks[g.ks_row(row, h) + lane / 8] = pair;
}
__device__ __forceinline__ void StoreRowK(const Kv8Geom& g, const Kv8Pools& p, int page0, size_t row, int h, int lane,
                                          float4 x) {
  if (g.kb == 4) Kv4StoreRowK(g, p, page0, row, h, lane, x);
  else Kv8StoreRowK(g, p, page0, row, h, lane, x);
}
// a channel's 16 keys of a tile to their place among the codes and stats
__device__ __forceinline__ void StoreTileV(const Kv8Geom& g, const Kv8Pools& p, int h, size_t pt, int d, const float (&x)[16]) {
  uint32_t stats;
  if (g.vb == 4) {
    uint2 codes;
    Kv4QuantTile(x, &codes, &stats);
    *reinterpret_cast<uint2*>(p.vq + g.vq_tile(h, pt) + size_t(d) * 2) = codes;
  } else {
    uint4 codes;
    Kv8QuantTile(x, &codes, &stats);
    *reinterpret_cast<uint4*>(p.vq + g.vq_tile(h, pt) + size_t(d) * 4) = codes;
  }
  p.vs[g.vs_tile(h, pt) + d] = stats;
}

// yah_kmean: thread (row group, channel); eight row groups, each summing its rows in order, then the groups in order
template <int DUMMY>
__global__ __launch_bounds__(256) void Kv8Kmean(const Kv8AppendArgs a) {
#pragma clang fp contract(off)
  const int s = blockIdx.y, t = threadIdx.x, cc = t % 32, grp = t / 32, W = a.g.W();
  const int c = blockIdx.x * 32 + cc;
  const int valid = a.n_valid != nullptr ? a.n_valid[s] : a.n_new;
  const int n = min(a.n_new, max(valid, 1));
  __shared__ float part[8][32];
  float acc = 0.0f;
  int r = grp;
  for (; r + 8 * 15 < n; r += 8 * 16) {  // sixteen loads in flight, added in the rows' order
    float x[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) x[j] = LoadSrc(a.k_src, (size_t(s) * a.n_new + r + 8 * j) * W + c, a.dtype);
#pragma unroll
    for (int j = 0; j < 16; ++j) acc = acc + TruncF16(x[j]);
  }
  for (; r < n; r += 8) acc = acc + TruncF16(LoadSrc(a.k_src, (size_t(s) * a.n_new + r) * W + c, a.dtype));
  part[grp][cc] = acc;
  __syncthreads();
  if (grp == 0) {
    float sum = 0.0f;
#pragma unroll
    for (int gi = 0; gi < 8; ++gi) sum = sum + part[gi][cc];
    a.p.km[size_t(PageOf(a, s, 0)) * W + c] = sum / static_cast<float>(n);
  }
}

// The decoder's append of one token: one wave per (kv head, sequence).
__global__ __launch_bounds__(64) void Kv8AppendToken(const Kv8AppendArgs a) {
  const int h = blockIdx.x, s = blockIdx.y, lane = threadIdx.x;
  int pos;
  if (RealTokens(a, s, &pos) < 1) return;
  const Kv8Geom& g = a.g;
  const int page = PageOf(a, s, pos), page0 = PageOf(a, s, 0);
  const size_t src = (size_t(s) * g.n_kv + h) * kKv8Dim + 4 * lane;
  const float4 k = Load4(a.k_src, src, a.dtype), v = Load4(a.v_src, src, a.dtype);
  StoreRowK(g, a.p, page0, size_t(page) * kKv8Page + pos % kKv8Page, h, lane, k);
  // V: the token's key of the open tile; on the tile's 16th key the tile is quantized into its place
  const int key = pos % 16;
  uint16_t* vo = a.p.vo + g.vo_head(page, h) + size_t(4 * lane) * 16;
  const float ve[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
  for (int e = 0; e < 4; ++e) vo[e * 16 + key] = F16Bits(ve[e]);
  if (key != 15) return;
  const size_t pt = size_t(page) * 16 + (pos / 16) % 16;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const uint4 lo = *reinterpret_cast<const uint4*>(vo + e * 16), hi = *reinterpret_cast<const uint4*>(vo + e * 16 + 8);
    const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
    float x[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) x[j] = WidenF16(static_cast<uint16_t>(w[j / 2] >> (16 * (j % 2))));
    x[15] = TruncF16(ve[e]);  // this lane's own store above
    StoreTileV(g, a.p, h, pt, 4 * lane + e, x);
  }
}

// The prefill's K rows: one workgroup of four waves per (token, sequence), the kv heads dealt to the waves.
__global__ __launch_bounds__(256) void Kv8AppendRowsK(const Kv8AppendArgs a) {
  const int i = blockIdx.x, s = blockIdx.y, wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  int p0;
  if (i >= RealTokens(a, s, &p0)) return;
  const Kv8Geom& g = a.g;
  const int pos = p0 + i, page = PageOf(a, s, pos), page0 = PageOf(a, s, 0);
  for (int h = wave; h < g.n_kv; h += 4) {
    const float4 k = Load4(a.k_src, ((size_t(s) * a.n_new + i) * g.n_kv + h) * kKv8Dim + 4 * lane, a.dtype);
    StoreRowK(g, a.p, page0, size_t(page) * kKv8Page + pos % kKv8Page, h, lane, k);
  }
}

// The prefill's V tiles: one workgroup per (16-key tile the chunk touches, sequence, kv head), thread = channel.
// Keys of the tile before the chunk's first are in the open tile; keys past the chunk's last real token repeat it.
__global__ __launch_bounds__(256) void Kv8AppendTilesV(const Kv8AppendArgs a) {
  const int s = blockIdx.y, h = blockIdx.z, d = threadIdx.x;
  int p0;
  const int nv = RealTokens(a, s, &p0);
  if (nv < 1) return;
  const Kv8Geom& g = a.g;
  const int last = p0 + nv - 1, t = p0 / 16 + blockIdx.x;
  if (16 * t > last) return;
  const int page = PageOf(a, s, 16 * t);
  uint16_t* vo = a.p.vo + g.vo_head(page, h) + size_t(d) * 16;
  float x[16];
  uint32_t open[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (16 * t < p0) {
    const uint4 lo = *reinterpret_cast<const uint4*>(vo), hi = *reinterpret_cast<const uint4*>(vo + 8);
    open[0] = lo.x, open[1] = lo.y, open[2] = lo.z, open[3] = lo.w, open[4] = hi.x, open[5] = hi.y, open[6] = hi.z, open[7] = hi.w;
  }
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const int pos = 16 * t + j;
    if (pos < p0) {
      x[j] = WidenF16(static_cast<uint16_t>(open[j / 2] >> (16 * (j % 2))));
    } else {
      const size_t i = static_cast<size_t>(min(pos, last) - p0);
      x[j] = TruncF16(LoadSrc(a.v_src, ((size_t(s) * a.n_new + i) * g.n_kv + h) * kKv8Dim + d, a.dtype));
    }
  }
  const size_t pt = size_t(page) * 16 + t % 16;
  StoreTileV(g, a.p, h, pt, d, x);
  if (t == last / 16) {  // yah_vseed: the newest tile stays open, keys past the last real token zero
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 16; j += 2) {
      const uint32_t b0 = 16 * t + j < p0 ? open[j / 2] & 0xFFFFu : (16 * t + j <= last ? F16Bits(x[j]) : 0u);
      const uint32_t b1 = 16 * t + j + 1 < p0 ? open[j / 2] >> 16 : (16 * t + j + 1 <= last ? F16Bits(x[j + 1]) : 0u);
      w[j / 2] = b0 | (b1 << 16);
    }
    *reinterpret_cast<uint4*>(vo) = uint4{w[0], w[1], w[2], w[3]};
    *reinterpret_cast<uint4*>(vo + 8) = uint4{w[4], w[5], w[6], w[7]};
  }
}

int FillArgs(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table, int32_t stride,
             const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs, int32_t n_new, const void* k_src,
             const void* v_src, int32_t dtype, Kv8AppendArgs* a) {
  if (const int st = CheckKv8Pools(g, pools)) return st;
  if (page_table == nullptr || k_src == nullptr || n_seqs <= 0 || n_new <= 0 || stride <= 0) return YAHKV_ERR_ARG;
  if (n_seqs > 65535 || g->n_kv_heads > 65535) return YAHKV_ERR_SHAPE;
  if (dtype != YAHKV_F32 && dtype != YAHKV_F16 && dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(k_src) | reinterpret_cast<uintptr_t>(v_src)) & 15) return YAHKV_ERR_ARG;
  *a = Kv8AppendArgs{MakeKv8Geom(*g), MakeKv8Pools(*pools), page_table, stride, start_pos, n_valid, n_new, k_src, v_src, dtype};
  return YAHKV_OK;
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" {

size_t yahkv_kv8_kq_bytes(const yahkv_geometry* g) {
  return CheckKv8Geometry(g) ? 0 : size_t(g->n_pages) * kKv8Page * g->n_kv_heads * MakeKv8Geom(*g).kq_head() * 4;
}
size_t yahkv_kv8_ks_bytes(const yahkv_geometry* g) {
  return CheckKv8Geometry(g) ? 0 : size_t(g->n_pages) * kKv8Page * g->n_kv_heads * MakeKv8Geom(*g).ks_head() * 4;
}
size_t yahkv_kv8_km_bytes(const yahkv_geometry* g) {
  return CheckKv8Geometry(g) ? 0 : size_t(g->n_pages) * g->n_kv_heads * kKv8Dim * 4;
}
size_t yahkv_kv8_vq_bytes(const yahkv_geometry* g) {
  return CheckKv8Geometry(g) ? 0 : size_t(g->n_pages) * 16 * g->n_kv_heads * kKv8Dim * MakeKv8Geom(*g).vq_dim() * 4;
}
size_t yahkv_kv8_vs_bytes(const yahkv_geometry* g) {
  return CheckKv8Geometry(g) ? 0 : size_t(g->n_pages) * 16 * g->n_kv_heads * kKv8Dim * 4;
}
size_t yahkv_kv8_vopen_bytes(const yahkv_geometry* g) {
  return CheckKv8Geometry(g) ? 0 : size_t(g->n_pages) * g->n_kv_heads * kKv8Dim * 16 * 2;
}

int yahkv_kv8_kmean(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                    int32_t page_table_stride, const int32_t* n_valid, int32_t n_seqs, int32_t n_rows,
                    const void* k_src, int32_t src_dtype, void* stream) {
  Kv8AppendArgs a;
  if (const int st = FillArgs(g, pools, page_table, page_table_stride, nullptr, n_valid, n_seqs, n_rows, k_src, k_src,
                              src_dtype, &a))
    return st;
  hipLaunchKernelGGL(Kv8Kmean<0>, dim3(a.g.W() / 32, n_seqs), dim3(256), 0, static_cast<hipStream_t>(stream), a);
  return LaunchStatus();
}

int yahkv_kv8_append(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                     int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs,
                     int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype, void* stream) {
  Kv8AppendArgs a;
  if (const int st = FillArgs(g, pools, page_table, page_table_stride, start_pos, n_valid, n_seqs, n_new, k_src, v_src,
                              src_dtype, &a))
    return st;
  if (start_pos == nullptr || v_src == nullptr) return YAHKV_ERR_ARG;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n_new == 1) {
    hipLaunchKernelGGL(Kv8AppendToken, dim3(g->n_kv_heads, n_seqs), dim3(64), 0, st, a);
    return LaunchStatus();
  }
  hipLaunchKernelGGL(Kv8AppendRowsK, dim3(n_new, n_seqs), dim3(256), 0, st, a);
  if (const int rc = LaunchStatus()) return rc;
  // a chunk that starts inside a tile touches one tile more than its length says
  hipLaunchKernelGGL(Kv8AppendTilesV, dim3((n_new + 15) / 16 + 1, n_seqs, g->n_kv_heads), dim3(256), 0, st, a);
  return LaunchStatus();
}

}  // extern "C"
