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

// The positions, counts and page table are read through the constant address space: nothing writes them while the
// kernel runs, and only then does the compiler use scalar loads, several of which go out together (as ordinary global
// loads each one waited for the one before, with a branch between).
typedef const int32_t __attribute__((address_space(4))) * ConstInts;
__device__ __forceinline__ ConstInts AsConst(const int32_t* p) { return (ConstInts)(reinterpret_cast<uintptr_t>(p)); }

// first position and number of real tokens of sequence s that lie inside the table; count 0: nothing to write
__device__ __forceinline__ int RealTokens(const Kv8AppendArgs& a, int s, int* p0) {
  const int start = AsConst(a.start_pos)[s];
  int nv = a.n_valid != nullptr ? min(AsConst(a.n_valid)[s], a.n_new) : a.n_new;
  *p0 = start;
  if (start < 0) return 0;
  const long long cap = static_cast<long long>(a.stride) * kKv8Page;
  if (start + static_cast<long long>(nv) > cap) nv = static_cast<int>(max(cap - start, 0ll));
  return max(nv, 0);
}
__device__ __forceinline__ int PageOf(const Kv8AppendArgs& a, int s, int pos) {
  return ClampPage(AsConst(a.table)[int64_t(s) * a.stride + pos / kKv8Page], a.g.n_pages);
}

// One K row of one kv head across a wave, four consecutive dims per lane: centre, scale per 128-dim half (32 lanes),
// codes, stores. `x`: the lane's four source values.
__device__ __forceinline__ void Kv8StoreRowK(const Kv8Geom& g, const Kv8Pools& p, float4 m, size_t row, int h, int lane,
                                             float4 x) {
#pragma clang fp contract(off)
  const float4 c = {TruncF16(x.x) - m.x, TruncF16(x.y) - m.y, TruncF16(x.z) - m.z, TruncF16(x.w) - m.w};
  float amax = fmaxf(fmaxf(fabsf(c.x), fabsf(c.y)), fmaxf(fabsf(c.z), fabsf(c.w)));
  amax = fmaxf(amax, LaneXor<1>(amax)), amax = fmaxf(amax, LaneXor<2>(amax)), amax = fmaxf(amax, LaneXor<4>(amax));
  amax = fmaxf(amax, LaneXor<8>(amax)), amax = fmaxf(amax, LaneXor<16>(amax));  // over the half's 32 lanes
  float inv;
  uint32_t pair;
  Kv8ScaleK(amax, &inv, &pair);
  p.kq[g.kq_row(row, h) + lane] = Kv8CodesK(c, inv);
  if (lane % 32 == 0) p.ks[g.ks_row(row, h) + lane / 32] = pair;
}
// the same for 4-bit K: rotated, 16 levels per 32-dim group (eight lanes), two lanes per dword
__device__ __forceinline__ void Kv4StoreRowK(const Kv8Geom& g, const Kv8Pools& p, float4 m, size_t row, int h, int lane,
                                             float4 x) {
#pragma clang fp contract(off)
  const float4 c = {TruncF16(x.x) - m.x, TruncF16(x.y) - m.y, TruncF16(x.z) - m.z, TruncF16(x.w) - m.w};
  uint32_t pair;
  float4 deq;
  uint32_t w = Kv4CodesK(c, lane, &pair, &deq);
  w |= LaneXorBits<1>(w);
  if (lane % 2 == 0) p.kq[g.kq_row(row, h) + lane / 2] = w;
  if (lane % 8 == 0) p.ks[g.ks_row(row, h) + lane / 8] = pair;
}
// `m`: the lane's four channel means (MeansK)
__device__ __forceinline__ void StoreRowK(const Kv8Geom& g, const Kv8Pools& p, float4 m, size_t row, int h, int lane,
                                          float4 x) {
  if (g.kb == 4) Kv4StoreRowK(g, p, m, row, h, lane, x);
  else Kv8StoreRowK(g, p, m, row, h, lane, x);
}
__device__ __forceinline__ float4 MeansK(const Kv8Geom& g, const Kv8Pools& p, int page0, int h, int lane) {
  return *reinterpret_cast<const float4*>(p.km + g.km_head(page0, h) + 4 * lane);
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

// yah_kmean: thread (row group, channel); eight row groups, each summing its rows in order, then the groups in order.
// SRC: the source rows' type, known when compiling: as a run-time value it put a branch behind every load, and the
// loads then went out one at a time, each waiting for the one before (2048 rows: 325 us; this way 32 are in flight).
template <int SRC>
__global__ __launch_bounds__(256) void Kv8Kmean(const Kv8AppendArgs a) {
#pragma clang fp contract(off)
  constexpr int kAhead = 32;
  const int s = blockIdx.y, t = threadIdx.x, cc = t % 32, grp = t / 32, W = a.g.W();
  const int c = blockIdx.x * 32 + cc;
  const int valid = a.n_valid != nullptr ? AsConst(a.n_valid)[s] : a.n_new;
  const int n = min(a.n_new, max(valid, 1));
  __shared__ float part[8][32];
  float acc = 0.0f;
  int r = grp;
  for (; r + 8 * (kAhead - 1) < n; r += 8 * kAhead) {  // added in the rows' order
    uint32_t x[kAhead];
#pragma unroll
    for (int j = 0; j < kAhead; ++j) x[j] = LoadRaw1(a.k_src, (size_t(s) * a.n_new + r + 8 * j) * W + c, SRC);
#pragma unroll
    for (int j = 0; j < kAhead; ++j) acc = acc + TruncF16(Widen1(x[j], SRC));
  }
  for (; r < n; r += 8) acc = acc + TruncF16(Widen1(LoadRaw1(a.k_src, (size_t(s) * a.n_new + r) * W + c, SRC), SRC));
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
  StoreRowK(g, a.p, MeansK(g, a.p, page0, h, lane), size_t(page) * kKv8Page + pos % kKv8Page, h, lane, k);
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

// The prefill's K rows: a workgroup of four waves takes kRowsPerGroup consecutive tokens of a sequence, the kv heads dealt
// to the waves; a wave asks for all its rows of a head, and for the head's means, before it works on the first (a row is
// a few round trips and 40 instructions: one row per workgroup left the memory system mostly waiting).
constexpr int kRowsPerGroup = 8;
static_assert(kRowsPerGroup <= kKv8Page, "a group's rows lie in at most two pages");
template <int SRC>
__device__ __forceinline__ void AppendRowsK(const Kv8AppendArgs& a, int i0, int s) {
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  int p0;
  const int nv = RealTokens(a, s, &p0);
  if (i0 >= nv) return;
  const Kv8Geom& g = a.g;
  // (the group's rows lie in at most two pages: both numbers now, not one per row between the rows' work)
  const int pos_a = p0 + i0, pos_b = p0 + min(i0 + kRowsPerGroup, nv) - 1;
  const int page0 = PageOf(a, s, 0), page_a = PageOf(a, s, pos_a), page_b = PageOf(a, s, pos_b);
  for (int h = wave; h < g.n_kv; h += 4) {
    uint4 raw[kRowsPerGroup];
#pragma unroll
    for (int r = 0; r < kRowsPerGroup; ++r) {
      const int i = min(i0 + r, nv - 1);
      raw[r] = LoadRaw4(a.k_src, ((size_t(s) * a.n_new + i) * g.n_kv + h) * kKv8Dim + 4 * lane, SRC);
    }
    const float4 m = MeansK(g, a.p, page0, h, lane);
#pragma unroll
    for (int r = 0; r < kRowsPerGroup; ++r) {
      if (i0 + r >= nv) break;
      const int pos = p0 + i0 + r, page = pos / kKv8Page == pos_a / kKv8Page ? page_a : page_b;
      StoreRowK(g, a.p, m, size_t(page) * kKv8Page + pos % kKv8Page, h, lane, Widen4(raw[r], SRC));
    }
  }
}

// The prefill's V tiles: one wave per (16-key tile the chunk touches, kv head), four channels per lane (a row of the
// source is then 8 or 16 bytes per lane; with a lane per channel the 2-byte loads kept the address units busier than
// the memory). Keys of the tile before the chunk's first are in the open tile; keys past the chunk's last real token
// repeat it.
__device__ __forceinline__ float Component(const float4& v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; }
template <int SRC>
__device__ __forceinline__ void AppendTileV(const Kv8AppendArgs& a, int item, int s) {
  const Kv8Geom& g = a.g;
  const int tile = item / g.n_kv, h = item % g.n_kv, d0 = 4 * (threadIdx.x % 64);
  int p0;
  const int nv = RealTokens(a, s, &p0);
  if (nv < 1) return;
  const int last = p0 + nv - 1, t = p0 / 16 + tile;
  if (16 * t > last) return;
  const int t_first = p0 / 16, t_last = last / 16;
  const bool reads_open = 16 * t_first < p0;
  const int page = PageOf(a, s, 16 * t), page_last = PageOf(a, s, 16 * t_last);
  uint16_t* vo = a.p.vo + g.vo_head(page, h) + size_t(d0) * 16;
  // all sixteen rows asked for at once (a key before the chunk's first asks for the first: its value is not used)
  uint4 raw[16];
  auto request = [&](int tt) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const size_t i = static_cast<size_t>(min(max(16 * tt + j, p0), last) - p0);
      raw[j] = LoadRaw4(a.v_src, ((size_t(s) * a.n_new + i) * g.n_kv + h) * kKv8Dim + d0, SRC);
    }
  };
  request(t);
  uint4 open[4][2] = {};
  if (16 * t < p0) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      open[e][0] = *reinterpret_cast<const uint4*>(vo + e * 16), open[e][1] = *reinterpret_cast<const uint4*>(vo + e * 16 + 8);
  }
  auto open_word = [&](int e, int w) -> uint32_t {  // keys 2 w, 2 w + 1 of channel d0 + e
    const uint4& q = open[e][w / 4];
    return w % 4 == 0 ? q.x : w % 4 == 1 ? q.y : w % 4 == 2 ? q.z : q.w;
  };
  // yah_vseed: the newest tile stays open, keys past the last real token zero. The open tile of a page is also what
  // the chunk's first tile reads when the chunk starts inside a tile, and first and newest tile can lie in one page: the
  // wave that reads the open tile is then also the one that writes it (each lane reads and writes its own channels'
  // bytes, in that order); left to the newest tile's wave the write could come before the read.
  const bool seeds = t == (reads_open ? t_first : t_last);
  const size_t pt = size_t(page) * 16 + t % 16;
  uint32_t stats[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {  // channel d0 + e
    float x[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const float from_open = WidenF16(static_cast<uint16_t>(open_word(e, j / 2) >> (16 * (j % 2))));
      x[j] = 16 * t + j < p0 ? from_open : TruncF16(Component(Widen4(raw[j], SRC), e));
    }
    if (g.vb == 4) {
      uint2 codes;
      Kv4QuantTile(x, &codes, &stats[e]);
      *reinterpret_cast<uint2*>(a.p.vq + g.vq_tile(h, pt) + size_t(d0 + e) * 2) = codes;
    } else {
      uint4 codes;
      Kv8QuantTile(x, &codes, &stats[e]);
      *reinterpret_cast<uint4*>(a.p.vq + g.vq_tile(h, pt) + size_t(d0 + e) * 4) = codes;
    }
    if (seeds && t == t_last) {
      uint32_t w[8];
#pragma unroll
      for (int j = 0; j < 16; j += 2) {
        const uint32_t b0 = 16 * t + j < p0 ? open_word(e, j / 2) & 0xFFFFu : (16 * t + j <= last ? F16Bits(x[j]) : 0u);
        const uint32_t b1 = 16 * t + j + 1 < p0 ? open_word(e, j / 2) >> 16 : (16 * t + j + 1 <= last ? F16Bits(x[j + 1]) : 0u);
        w[j / 2] = b0 | (b1 << 16);
      }
      *reinterpret_cast<uint4*>(vo + e * 16) = uint4{w[0], w[1], w[2], w[3]};
      *reinterpret_cast<uint4*>(vo + e * 16 + 8) = uint4{w[4], w[5], w[6], w[7]};
    }
  }
  *reinterpret_cast<uint4*>(a.p.vs + g.vs_tile(h, pt) + d0) = uint4{stats[0], stats[1], stats[2], stats[3]};
  if (!seeds || t == t_last) return;
  // the newest tile lies wholly inside the chunk: its rows once more
  request(t_last);
  vo = a.p.vo + g.vo_head(page_last, h) + size_t(d0) * 16;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    uint32_t w[8];
#pragma unroll
    for (int j = 0; j < 16; j += 2) {
      const uint32_t b0 = 16 * t_last + j <= last ? F16Bits(TruncF16(Component(Widen4(raw[j], SRC), e))) : 0u;
      const uint32_t b1 = 16 * t_last + j + 1 <= last ? F16Bits(TruncF16(Component(Widen4(raw[j + 1], SRC), e))) : 0u;
      w[j / 2] = b0 | (b1 << 16);
    }
    *reinterpret_cast<uint4*>(vo + e * 16) = uint4{w[0], w[1], w[2], w[3]};
    *reinterpret_cast<uint4*>(vo + e * 16 + 8) = uint4{w[4], w[5], w[6], w[7]};
  }
}

// A chunk's K rows and V tiles in one launch (they are independent): blocks [0, k_groups) take the K rows, the waves of
// the rest one (tile, kv head) each, kv head fastest. SRC: the source rows' type (see Kv8Kmean).
template <int SRC>
__global__ __launch_bounds__(256) void Kv8AppendChunk(const Kv8AppendArgs a, int k_groups) {
  const int b = blockIdx.x, s = blockIdx.y;
  if (b < k_groups) AppendRowsK<SRC>(a, b * kRowsPerGroup, s);
  else AppendTileV<SRC>(a, (b - k_groups) * 4 + static_cast<int>(threadIdx.x / 64), s);
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
  const dim3 grid(a.g.W() / 32, n_seqs);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (src_dtype == YAHKV_F32) hipLaunchKernelGGL(Kv8Kmean<YAHKV_F32>, grid, dim3(256), 0, st, a);
  else if (src_dtype == YAHKV_F16) hipLaunchKernelGGL(Kv8Kmean<YAHKV_F16>, grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL(Kv8Kmean<YAHKV_BF16>, grid, dim3(256), 0, st, a);
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
  // a chunk that starts inside a tile touches one tile more than its length says
  const int k_groups = (n_new + kRowsPerGroup - 1) / kRowsPerGroup;
  const long long blocks = k_groups + (static_cast<long long>((n_new + 15) / 16 + 1) * g->n_kv_heads + 3) / 4;
  if (blocks > 0x7fffffffll) return YAHKV_ERR_SHAPE;
  const dim3 grid(static_cast<unsigned>(blocks), n_seqs);
  if (src_dtype == YAHKV_F32) hipLaunchKernelGGL(Kv8AppendChunk<YAHKV_F32>, grid, dim3(256), 0, st, a, k_groups);
  else if (src_dtype == YAHKV_F16) hipLaunchKernelGGL(Kv8AppendChunk<YAHKV_F16>, grid, dim3(256), 0, st, a, k_groups);
  else hipLaunchKernelGGL(Kv8AppendChunk<YAHKV_BF16>, grid, dim3(256), 0, st, a, k_groups);
  return LaunchStatus();
}

}  // extern "C"
