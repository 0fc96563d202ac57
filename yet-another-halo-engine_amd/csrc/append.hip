// Token append: block-quantize K and V rows and scatter them into their pages, optionally with the head RMSNorm and
// NeoX RoPE of K (and of the queries) fused in; and the inverse gather used by tests.
//
// Placement follows the reference's page mapping (engine/gpu/loom/tools/gen_kvq.py:48-71): token at position p goes
// to page table[p / PT] (clamped into the pool), slot p % PT; positions are clamped to the table
// (gen_decode_attn.py:59-63). The quantizers are in quant.hpp.
//
// The fused form follows the reference's decode kernel (engine/gpu/loom/yah_fused_qk_rope_f32.loom:1-10, Q branch
// :96-146, K branch :147-241) and its batched, paged rewrite for prefill chunks
// (engine/gpu/loom/tools/emit_prefill_pp.py:31-111): per head
//   inv_rms = rsqrt(sum_i x[i]^2 / head_dim + eps); normed[i] = (x[i] * inv_rms) * weight[i]
//   angle(p) = pos * (1 / theta^(2 p / rotary_dim)), p < half = rotary_dim / 2
//   out[p] = normed[p] cos - normed[p + half] sin; out[p + half] = normed[p] sin + normed[p + half] cos
// and dims at or past rotary_dim are only normalised. The angle uses the token's position as given; the page slot
// uses the position clamped to the table, as in the reference (:89-94). What the reference stores as f16 rows is
// stored here as q8_0 / q4_0 blocks: the rotated K never makes a round trip through memory as f32.
#include "common.hpp"
#include "quant.hpp"

namespace yahkv {
namespace {

struct RopeArgs {
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
  const float* k_weight;
  const float* q_weight;
  float theta, eps;
  int32_t rotary_dim;
  const void* q_src;  // [n_seqs][n_new][n_q][D] of src_dtype, or null
  void* q_out;        // same shape, of q_out_dtype
  int32_t q_out_dtype;
  float* k_out;       // [n_seqs][n_new][H][D] f32 or null: the rotated K rows, for callers that want them
  int32_t per_xcd;    // AppendRows: tokens per XCD and sequence (a multiple of the page), or 0: tokens in order
  int32_t skip_v;     // AppendRows: the V rows are left to another launch (AppendPages with skip_k)
  int32_t skip_k;     // AppendPages: V only
};

__device__ __forceinline__ void Store4(void* dst, size_t i, int dtype, float4 v) {
  if (dtype == YAHKV_F32) {
    *reinterpret_cast<float4*>(static_cast<float*>(dst) + i) = v;
    return;
  }
  uint32_t lo, hi;
  if (dtype == YAHKV_F16) {
    typedef _Float16 h2v __attribute__((ext_vector_type(2)));
    lo = __builtin_bit_cast(uint32_t, h2v{static_cast<_Float16>(v.x), static_cast<_Float16>(v.y)});
    hi = __builtin_bit_cast(uint32_t, h2v{static_cast<_Float16>(v.z), static_cast<_Float16>(v.w)});
  } else {
    typedef __bf16 b2v __attribute__((ext_vector_type(2)));
    lo = __builtin_bit_cast(uint32_t, b2v{static_cast<__bf16>(v.x), static_cast<__bf16>(v.y)});
    hi = __builtin_bit_cast(uint32_t, b2v{static_cast<__bf16>(v.z), static_cast<__bf16>(v.w)});
  }
  *reinterpret_cast<uint2*>(static_cast<uint16_t*>(dst) + i) = uint2{lo, hi};
}

// One workgroup of four wavefronts per token. With ROPE, the token's angles (they depend on the position and the
// pair, not on the head) are computed once into LDS; without, K rows are quantized as they are (plain append) and
// there are no query rows. The token's rows of head_dim values (its H K heads, its H V heads, then its
// query heads) are dealt to the wavefronts in turn; a row lies across a wavefront, four consecutive dims per lane, so
// every load and store is 16 (or 8) bytes per lane, the sum of squares and the block maxima are DPP reductions, and
// the partner of a rotated pair comes through one lane shuffle: rows never go through LDS. A wavefront issues the
// loads of all its rows (up to eight at a time) before it works on the first; for that the loads must not sit behind
// branches, so the source rows' type SRC is known when compiling (as in AppendPages: with the type a run-time value
// each load waited for the one before) and a row or lane that has nothing to load asks for an address that exists.
constexpr int kRopeWaves = 4, kRowsInFlight = 8;
template <int FMT, bool ROPE, int SRC>
__global__ __launch_bounds__(64 * kRopeWaves) void AppendRows(const RopeArgs a) {
#pragma clang fp contract(off)
  const Geom g = a.g;
  const int H = g.n_kv, PT = g.pt, D = g.hd, NQ = a.q_src != nullptr ? g.n_q : 0;
  // (with a.skip_v the token's rows are its K heads and its query heads: row numbers H .. 2 H - 1 are passed over)
  const int rows_per_token = (a.skip_v ? H : 2 * H) + NQ;
  auto row_of = [&](int r) -> int { return a.skip_v && r >= H ? r + H : r; };
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  // Token i of sequence s. Workgroup b of a dispatch runs on XCD b % 8, and V's codes are single bytes of the
  // transposed page: with a long chunk's tokens dealt to the workgroups in order, every line of a page would be put
  // together from bytes in eight L2 caches, each of which writes its part back on its own. a.per_xcd > 0: workgroups
  // b, b + 8, ... take per_xcd consecutive tokens (whole pages), so a page's bytes meet in one L2.
  int i = int(blockIdx.x % a.n_new), s = int(blockIdx.x / a.n_new);
  if (a.per_xcd > 0) {
    const int span = 8 * a.per_xcd, r = int(blockIdx.x % span);
    s = int(blockIdx.x / span), i = (r % 8) * a.per_xcd + r / 8;
    if (i >= a.n_new) return;
  }
  const int nv = a.n_valid != nullptr ? min(a.n_valid[s], a.n_new) : a.n_new;
  if (i >= nv) return;  // padding row of a short chunk
  const int start = a.start_pos[s], pos_raw = start + i, last_pos = a.stride * PT - 1;
  const int pos = min(max(pos_raw, 0), last_pos);
  // Where several tokens of the call clamp to the table's first or last slot, the one a loop over the tokens would
  // leave there writes it (AppendPages' token_at); the others only produce their query rows and rotated K rows.
  const bool owns_slot = pos_raw >= last_pos ? i == nv - 1 : (pos_raw <= 0 ? i == min(nv - 1, -start) : true);
  const int page = ClampPage(a.table[int64_t(s) * a.stride + pos / PT], g.n_pages);
  const int t = pos % PT;

  __shared__ __align__(16) float cs[128], sn[128];  // rotary_dim / 2 <= 128
  const int rot = a.rotary_dim, half = rot / 2;
  const float posf = static_cast<float>(pos_raw);
  if (ROPE) {
    for (int p = threadIdx.x; p < half; p += 64 * kRopeWaves) {
      const float inv_freq = 1.0f / powf(a.theta, (2.0f * static_cast<float>(p)) / static_cast<float>(rot));
      float sv, cv;
      sincosf(posf * inv_freq, &sv, &cv);
      cs[p] = cv, sn[p] = sv;
    }
    __syncthreads();
  }
  const int d0 = 4 * lane;  // this lane's four dims of every row
  const bool has = d0 < D;
  // This lane's part of the rotation, the same for every row: element e = d0 + j is the first of its pair
  // (e < half: out = x c - partner s, partner = e + half), the second (half <= e < rot: out = partner s + x c,
  // partner = e - half) or past the rotated dims. rotary_dim / 2 is a multiple of 4 (checked by the entry point), so
  // the four partners lie in one lane.
  float c4[4] = {1.0f, 1.0f, 1.0f, 1.0f}, s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  int partner_lane = lane;
  if (ROPE && has && d0 < rot) {
    const bool first = d0 < half;
    partner_lane = first ? lane + half / 4 : lane - half / 4;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int p = first ? d0 + j : d0 + j - half;
      c4[j] = cs[p];
      s4[j] = first ? -sn[p] : sn[p];
    }
  }
  float4 wk = {1.0f, 1.0f, 1.0f, 1.0f}, wq = wk;  // this lane's norm weights
  if (ROPE && a.k_weight != nullptr && has) wk = *reinterpret_cast<const float4*>(a.k_weight + d0);
  if (ROPE && a.q_weight != nullptr && has) wq = *reinterpret_cast<const float4*>(a.q_weight + d0);
  // source of row `row` of the token and its element offset
  auto source = [&](int row, const void** src, size_t* off) {
    const size_t tok = size_t(s) * a.n_new + i;
    if (row < H) *src = a.k_src, *off = (tok * H + row) * D;
    else if (row < 2 * H) *src = a.v_src, *off = (tok * H + (row - H)) * D;
    else *src = a.q_src, *off = (tok * g.n_q + (row - 2 * H)) * D;
  };
  for (int first_row = wave; first_row < rows_per_token; first_row += kRopeWaves * kRowsInFlight) {
    uint4 raw[kRowsInFlight];
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
      const void* src;
      size_t off;
      source(row_of(min(first_row + kRopeWaves * j, rows_per_token - 1)), &src, &off);
      raw[j] = LoadRaw4(src, off + (has ? d0 : 0), SRC);
    }
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
      if (first_row + kRopeWaves * j >= rows_per_token) break;
      const int row = row_of(first_row + kRopeWaves * j);
      const bool is_v = row >= H && row < 2 * H, is_q = row >= 2 * H;
      float4 v = Widen4(raw[j], SRC);
      if (!has) v = float4{0.0f, 0.0f, 0.0f, 0.0f};
      if (ROPE && !is_v) {
        const float ss = WaveSum(v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w);
        const float inv_rms = 1.0f / sqrtf(ss / static_cast<float>(D) + a.eps);
        const float4 w = is_q ? wq : wk;
        v = float4{(v.x * inv_rms) * w.x, (v.y * inv_rms) * w.y, (v.z * inv_rms) * w.z, (v.w * inv_rms) * w.w};
        const float px = __shfl(v.x, partner_lane, 64), py = __shfl(v.y, partner_lane, 64);
        const float pz = __shfl(v.z, partner_lane, 64), pw = __shfl(v.w, partner_lane, 64);
        // first of a pair: x c - partner s; second: partner s + x c (s4 carries the sign); past rot: c = 1, s = 0
        v = float4{v.x * c4[0] + px * s4[0], v.y * c4[1] + py * s4[1], v.z * c4[2] + pz * s4[2],
                   v.w * c4[3] + pw * s4[3]};
      }
      const void* src;
      size_t off;
      source(row, &src, &off);
      if (is_q) {
        if (has) Store4(a.q_out, off + d0, a.q_out_dtype, v);
        continue;
      }
      if (!is_v && a.k_out != nullptr && has) *reinterpret_cast<float4*>(a.k_out + off + d0) = v;
      // quantize: block b = lanes 8 b .. 8 b + 7
      const int h = is_v ? row - H : row, lb = lane % 8;
      uint16_t scale;
      const uint32_t codes = FMT == 8 ? QuantizeLanesQ8(v, &scale) : QuantizeLanesQ4(v, lb, &scale);
      if (!has || !owns_slot) continue;
      if (!is_v)
        StoreRowK<FMT>(a.pools, g, page, h, t, lane, codes, scale);
      else
        StoreRowV<FMT>(a.pools, g, page, h, t, lane, codes, scale);
    }
  }
}

// Chunks: one workgroup per (sequence, page touched by the chunk, kv head). A token at a time per wavefront, the rows
// are quantized exactly as above, but the codes and scales go to an LDS image of the page's (page, head) regions, and
// the image leaves for HBM in 16-byte pieces once the page's tokens are done. Token by token the V codes would be
// single bytes 64 bytes apart (V lies transposed, [dim][token], so that decode reads 16 tokens of a dim at once) and
// every K block a 32-byte piece; page by page they are whole lines.
// Positions clamp to the table as everywhere (gen_decode_attn.py:59-63); where several tokens of a chunk clamp to
// the same slot (the first or the last of the table), the last token wins, as in a loop over the tokens.
constexpr int kPageWaves = 4;
constexpr int kPageAppendMin = 8;  // tokens per sequence from which a call is treated as a chunk
// SRC: the source rows' type, known when compiling (as a run-time value it put a three-way branch around every
// row's conversion).
template <int FMT, int SRC>
__global__ __launch_bounds__(64 * kPageWaves) void AppendPages(const RopeArgs a) {
#pragma clang fp contract(off)
  const Geom g = a.g;
  const int NB = g.nb(), H = g.n_kv, PT = g.pt, D = g.hd;
  constexpr int KB = FMT == 8 ? 32 : 16;                 // bytes of K codes per token and block
  const int v_rows = FMT == 8 ? D : NB * 16;             // byte rows of the V image, PT bytes each
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, h = blockIdx.y, s = blockIdx.z;
  const int nv = a.n_valid != nullptr ? min(max(a.n_valid[s], 0), a.n_new) : a.n_new;
  if (nv <= 0) return;
  const int start = a.start_pos[s], last_pos = a.stride * PT - 1;
  const int p_first = min(max(start, 0), last_pos), p_last = min(max(start + nv - 1, 0), last_pos);
  const int pi = p_first / PT + blockIdx.x;
  if (pi > p_last / PT) return;
  const int t_lo = max(p_first, pi * PT) - pi * PT, t_hi = min(p_last, pi * PT + PT - 1) - pi * PT + 1;
  const int page = ClampPage(a.table[int64_t(s) * a.stride + pi], g.n_pages);
  // the token of the chunk that ends up at position pos (the last one, where several clamp to it)
  auto token_at = [&](int pos) -> int {
    if (pos == last_pos && start + nv - 1 >= last_pos) return nv - 1;
    if (pos == 0 && start <= 0) return min(nv - 1, -start);
    return pos - start;
  };

  __shared__ __align__(16) uint8_t lk[8 * 64 * 32], lv[256 * (64 + 4)];  // images of the K and V code regions
  __shared__ __align__(16) uint16_t lks[64 * 8], lvs[8 * 64];      // and of the scale regions
  const int d0 = 4 * lane, b = lane / 8, lb = lane % 8;
  const bool has = d0 < D;
  // A wavefront takes four consecutive tokens at a time (their rows in flight together): a lane then holds, for each
  // of its four dims, the codes of four neighbouring tokens, which is one dword of the V image instead of four bytes.
  // (The image's rows are padded by a dword: with rows of exactly PT bytes the 64 lanes of such a store would all
  // hit one LDS bank.)
  // The rows of the wave's next four tokens are requested before the current four are quantized.
  uint4 rk[4], rv[4];
  auto request = [&](int q) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int t = 4 * q + j;
      rk[j] = rv[j] = uint4{0u, 0u, 0u, 0u};  // reads as 0.0 in every source type
      if (t >= t_lo && t < t_hi && has) {
        const size_t row = ((size_t(s) * a.n_new + token_at(pi * PT + t)) * H + h) * D;
        rv[j] = LoadRaw4(a.v_src, row + d0, SRC);
        if (!a.skip_k) rk[j] = LoadRaw4(a.k_src, row + d0, SRC);
      }
    }
  };
  if (4 * (t_lo / 4 + wave) < t_hi) request(t_lo / 4 + wave);
  for (int q = t_lo / 4 + wave; 4 * q < t_hi; q += kPageWaves) {
    float4 kx[4], vx[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) kx[j] = Widen4(rk[j], SRC), vx[j] = Widen4(rv[j], SRC);
    if (4 * (q + kPageWaves) < t_hi) request(q + kPageWaves);
    uint32_t vc[4];
    if constexpr (FMT == 8) {
      // Eight rows are in flight (K and V of four tokens) and a block has eight lanes: lane lb of a block takes row
      // lb's amax and does the two divisions for it (the same operations on the same values, so the same bits),
      // instead of every lane doing them for every row; the reciprocals go back through lane shuffles.
      float am[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) am[j] = BlockAmaxQ8(kx[j]), am[4 + j] = BlockAmaxQ8(vx[j]);
      float mine = am[0];
#pragma unroll
      for (int r = 1; r < 8; ++r) mine = lb == r ? am[r] : mine;
      float inv;
      uint16_t sc;
      ScaleQ8(mine, &inv, &sc);
      {
        const int t = 4 * q + lb % 4;  // row lb is K (lb < 4) or V of this token
        if (has && t >= t_lo && t < t_hi) {
          if (lb < 4) lks[t * NB + b] = sc;
          else lvs[b * PT + t] = sc;
        }
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int t = 4 * q + j;
        const uint32_t kc = CodesLanesQ8(kx[j], __shfl(inv, (lane & ~7) | j, 64));
        vc[j] = CodesLanesQ8(vx[j], __shfl(inv, (lane & ~7) | (4 + j), 64));
        if (!has || t < t_lo || t >= t_hi) continue;
        *reinterpret_cast<uint32_t*>(&lk[(b * PT + t) * KB + 4 * lb]) = kc;
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int t = 4 * q + j;
        uint16_t ksc, vsc;
        const uint32_t kc = QuantizeLanesQ4(kx[j], lb, &ksc);
        vc[j] = QuantizeLanesQ4(vx[j], lb, &vsc);
        if (!has || t < t_lo || t >= t_hi) continue;
        if (lb == 0) lks[t * NB + b] = ksc, lvs[b * PT + t] = vsc;
        if (lb < 4) *reinterpret_cast<uint32_t*>(&lk[(b * PT + t) * KB + 4 * lb]) = kc;
      }
    }
    if (has && (FMT == 8 || lb < 4)) {
      const int r0 = FMT == 8 ? d0 : b * 16 + 4 * lb;  // this lane's four byte rows of the V image
#pragma unroll
      for (int e = 0; e < 4; ++e)
        *reinterpret_cast<uint32_t*>(&lv[(r0 + e) * (PT + 4) + 4 * q]) =
            ((vc[0] >> (8 * e)) & 0xFF) | (((vc[1] >> (8 * e)) & 0xFF) << 8) | (((vc[2] >> (8 * e)) & 0xFF) << 16) |
            (((vc[3] >> (8 * e)) & 0xFF) << 24);
    }
  }
  __syncthreads();
  // ---- the images' written parts to the pools
  const size_t ph = size_t(page) * H + h;
  const int n_t = t_hi - t_lo, tid = threadIdx.x, NT = 64 * kPageWaves;
  const int lg_pt = __builtin_ctz(static_cast<unsigned>(PT));  // pages are 16, 32 or 64 tokens
  if (!a.skip_k) {  // K codes: per block the tokens' pieces are contiguous
    uint8_t* dst = a.pools.kq + ph * (size_t(NB) * PT * KB);
    if (n_t == PT) {  // a whole page (most of a chunk's): the region as it lies, no division by a run-time value
      for (int u = tid; u < (NB * KB / 16) << lg_pt; u += NT)
        *reinterpret_cast<uint4*>(dst + u * 16) = *reinterpret_cast<const uint4*>(&lk[u * 16]);
    } else {
      const int per_block = n_t * KB / 16;
      for (int u = tid; u < NB * per_block; u += NT) {
        const int off = ((u / per_block) * PT + t_lo) * KB + (u % per_block) * 16;
        *reinterpret_cast<uint4*>(dst + off) = *reinterpret_cast<const uint4*>(&lk[off]);
      }
    }
  }
  if (!a.skip_k) {  // K scales: [token][block], 8 bytes at a time
    uint8_t* dst = reinterpret_cast<uint8_t*>(a.pools.ks) + ph * (size_t(PT) * NB * 2);
    for (int u = tid; u < n_t * NB / 4; u += NT) {
      const int off = t_lo * NB * 2 + u * 8;
      *reinterpret_cast<uint2*>(dst + off) = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint8_t*>(lks) + off);
    }
  }
  uint8_t* vdst = a.pools.vq + ph * (size_t(v_rows) * PT);
  uint16_t* sdst = a.pools.vs + ph * (size_t(NB) * PT);
  if (n_t == PT) {  // a whole page: both V regions are contiguous
    for (int u = tid; u < (v_rows << lg_pt) / 16; u += NT) {
      const uint32_t* src = reinterpret_cast<const uint32_t*>(&lv[((u * 16) >> lg_pt) * (PT + 4) + ((u * 16) & (PT - 1))]);
      *reinterpret_cast<uint4*>(vdst + u * 16) = uint4{src[0], src[1], src[2], src[3]};
    }
    for (int u = tid; u < NB * PT / 8; u += NT)
      *reinterpret_cast<uint4*>(sdst + u * 8) = *reinterpret_cast<const uint4*>(&lvs[u * 8]);
  } else {  // the chunk's first or last page: the tokens' bytes of every row
    for (int u = tid; u < v_rows * n_t; u += NT) {
      const int r = u / n_t, t = t_lo + u % n_t;
      vdst[r * PT + t] = lv[r * (PT + 4) + t];
    }
    for (int u = tid; u < NB * n_t; u += NT) {
      const int off = (u / n_t) * PT + t_lo + u % n_t;
      sdst[off] = lvs[off];
    }
  }
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

namespace {
int CheckAppend(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                int32_t page_table_stride, const int32_t* start_pos, int32_t n_seqs, int32_t n_new, const void* k_src,
                const void* v_src, int32_t src_dtype) {
  if (const int st = CheckPools(g, pools)) return st;
  if (page_table == nullptr || start_pos == nullptr || k_src == nullptr || v_src == nullptr) return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || n_new <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (src_dtype != YAHKV_F32 && src_dtype != YAHKV_F16 && src_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(k_src) | reinterpret_cast<uintptr_t>(v_src)) & 15) return YAHKV_ERR_ARG;
  if (int64_t(n_seqs) * n_new > 0x7FFFFFFF) return YAHKV_ERR_SHAPE;
  return YAHKV_OK;
}
}  // namespace

namespace {
// AppendRows for the pools' format and the source rows' type (the kernel is compiled for each pair)
// AppendPages likewise: one workgroup per (page the chunk touches, kv head, sequence)
void LaunchPages(int32_t format, int32_t src_dtype, int32_t n_seqs, int32_t n_new, hipStream_t st, const RopeArgs& a) {
  const dim3 grid(static_cast<unsigned>((n_new + a.g.pt - 2) / a.g.pt + 1), static_cast<unsigned>(a.g.n_kv),
                  static_cast<unsigned>(n_seqs));
  const dim3 block(64 * kPageWaves);
  if (format == YAHKV_Q8_0) {
    if (src_dtype == YAHKV_F32) hipLaunchKernelGGL((AppendPages<8, YAHKV_F32>), grid, block, 0, st, a);
    else if (src_dtype == YAHKV_F16) hipLaunchKernelGGL((AppendPages<8, YAHKV_F16>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((AppendPages<8, YAHKV_BF16>), grid, block, 0, st, a);
  } else {
    if (src_dtype == YAHKV_F32) hipLaunchKernelGGL((AppendPages<4, YAHKV_F32>), grid, block, 0, st, a);
    else if (src_dtype == YAHKV_F16) hipLaunchKernelGGL((AppendPages<4, YAHKV_F16>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((AppendPages<4, YAHKV_BF16>), grid, block, 0, st, a);
  }
}
template <bool ROPE>
void LaunchRows(int32_t format, int32_t src_dtype, dim3 grid, hipStream_t st, const RopeArgs& a) {
  const dim3 block(64 * kRopeWaves);
  if (format == YAHKV_Q8_0) {
    if (src_dtype == YAHKV_F32) hipLaunchKernelGGL((AppendRows<8, ROPE, YAHKV_F32>), grid, block, 0, st, a);
    else if (src_dtype == YAHKV_F16) hipLaunchKernelGGL((AppendRows<8, ROPE, YAHKV_F16>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((AppendRows<8, ROPE, YAHKV_BF16>), grid, block, 0, st, a);
  } else {
    if (src_dtype == YAHKV_F32) hipLaunchKernelGGL((AppendRows<4, ROPE, YAHKV_F32>), grid, block, 0, st, a);
    else if (src_dtype == YAHKV_F16) hipLaunchKernelGGL((AppendRows<4, ROPE, YAHKV_F16>), grid, block, 0, st, a);
    else hipLaunchKernelGGL((AppendRows<4, ROPE, YAHKV_BF16>), grid, block, 0, st, a);
  }
}
}  // namespace

extern "C" int yahkv_append(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                            int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid,
                            int32_t n_seqs, int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype,
                            void* stream) {
  if (const int st = CheckAppend(g, pools, page_table, page_table_stride, start_pos, n_seqs, n_new, k_src, v_src,
                                 src_dtype))
    return st;
  RopeArgs a{};
  a.g = MakeGeom(*g), a.pools = MakePools(*pools), a.table = page_table, a.stride = page_table_stride;
  a.start_pos = start_pos, a.n_valid = n_valid, a.n_seqs = n_seqs, a.n_new = n_new, a.k_src = k_src, a.v_src = v_src;
  a.src_dtype = src_dtype, a.rotary_dim = 8, a.theta = 1.0f;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n_new >= kPageAppendMin && n_seqs <= 65535) {  // a chunk: page by page (the grid's z extent is the batch)
    LaunchPages(g->format, src_dtype, n_seqs, n_new, st, a);
    return LaunchStatus();
  }
  const dim3 grid(static_cast<unsigned>(n_seqs) * static_cast<unsigned>(n_new));
  LaunchRows<false>(g->format, src_dtype, grid, st, a);
  return LaunchStatus();
}

extern "C" int yahkv_append_rope(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                 int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid,
                                 int32_t n_seqs, int32_t n_new, const void* k_src, const void* v_src,
                                 int32_t src_dtype, const yahkv_rope* rope, const void* q_src, void* q_out,
                                 int32_t q_out_dtype, float* k_out, void* stream) {
  if (const int st = CheckAppend(g, pools, page_table, page_table_stride, start_pos, n_seqs, n_new, k_src, v_src,
                                 src_dtype))
    return st;
  if (rope == nullptr) return YAHKV_ERR_ARG;
  if ((q_src == nullptr) != (q_out == nullptr)) return YAHKV_ERR_ARG;
  if (q_src != nullptr && q_out_dtype != YAHKV_F32 && q_out_dtype != YAHKV_F16 && q_out_dtype != YAHKV_BF16)
    return YAHKV_ERR_ARG;
  const Geom m = MakeGeom(*g);
  if (rope->rotary_dim < 8 || rope->rotary_dim > m.hd || rope->rotary_dim % 8 != 0) return YAHKV_ERR_ARG;
  if (!(rope->theta > 0.0f) || !(rope->eps >= 0.0f)) return YAHKV_ERR_ARG;
  RopeArgs a{};
  a.g = m, a.pools = MakePools(*pools), a.table = page_table, a.stride = page_table_stride, a.start_pos = start_pos;
  a.n_valid = n_valid, a.n_seqs = n_seqs, a.n_new = n_new, a.k_src = k_src, a.v_src = v_src, a.src_dtype = src_dtype;
  a.k_weight = rope->k_weight, a.q_weight = rope->q_weight, a.theta = rope->theta, a.eps = rope->eps;
  a.rotary_dim = rope->rotary_dim, a.q_src = q_src, a.q_out = q_out, a.q_out_dtype = q_out_dtype, a.k_out = k_out;
  const int64_t tokens = int64_t(n_seqs) * n_new;
  if (tokens > 0x7FFFFFFF) return YAHKV_ERR_SHAPE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (n_new >= kPageAppendMin && n_seqs <= 65535) {
    // A chunk: V page by page, as the plain append takes it (whole lines from an image of the page, where the
    // token's workgroup would store V's codes byte by byte into the transposed page), K and the query rows by token.
    RopeArgs v = a;
    v.skip_k = 1;
    LaunchPages(g->format, src_dtype, n_seqs, n_new, st, v);
    if (const int rc = LaunchStatus()) return rc;
    a.skip_v = 1;
  }
  int64_t blocks = tokens;
  if (n_new >= 8 * m.pt) {  // a long chunk: a page's tokens to one XCD (see AppendRows)
    a.per_xcd = ((n_new + 7) / 8 + m.pt - 1) / m.pt * m.pt;
    blocks = int64_t(n_seqs) * 8 * a.per_xcd;
    if (blocks > 0x7FFFFFFF) return YAHKV_ERR_SHAPE;
  }
  LaunchRows<true>(g->format, src_dtype, dim3(static_cast<unsigned>(blocks)), st, a);
  return LaunchStatus();
}

extern "C" int yahkv_gather_blocks(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row,
                                   int32_t n_tokens, void* dst_k, void* dst_v, void* stream) {
  if (const int st = CheckPools(g, pools)) return st;
  if (table_row == nullptr || dst_k == nullptr || dst_v == nullptr || n_tokens <= 0) return YAHKV_ERR_ARG;
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
