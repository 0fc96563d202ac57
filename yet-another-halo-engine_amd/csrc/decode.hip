// Paged GQA decode attention over block-quantized K/V: split-K over 64-token tiles, then a merge.
//
// Structure follows the reference's decode attention (engine/gpu/loom/tools/gen_decode_attn.py): `part` computes one
// partial (M, l, acc) per slice of the context for the query heads of one kv head (:97-335, quantized :576-1040),
// `reduce` merges the partials: out = (sum_s e^(M_s - M) acc_s) / (sum_s e^(M_s - M) l_s) * sigmoid(gate) (:338-411).
// Keys at or past the sequence length are masked (key < pos + 1, :145,167); the "minus infinity" is the finite
// -FLT_MAX the reference uses (:357), so that no inf - inf can appear.
#include <algorithm>

#include "common.hpp"

namespace yahkv {
namespace {

constexpr float kNegMax = -3.4028234663852886e+38f;
constexpr int kTile = 64;     // tokens per tile: one wavefront, one token per lane in the score phase
constexpr int kWaves = 4;
constexpr int kMaxGroup = 8;  // query heads per kv head

struct DecodeArgs {
  Geom g;
  Pools pools;
  const int32_t* table;
  int32_t stride;
  const int32_t* seq_len;
  int32_t n_seqs, max_len;  // max_len already clamped to stride * PT
  const void* q;
  int32_t q_dtype;
  float scale;
  const float* gate;
  float* out;
  float* acc;  // [n_seqs][H][n_splits][G][D]
  float* ml;   // [n_seqs][H][n_splits][G][2]
  int32_t n_splits, tiles_per_split;
};

__device__ __forceinline__ float WaveMax(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float WaveSum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// Dimension k (< D / 64) of lane `lane`: q8_0 keeps a lane's dims contiguous; q4_0 pairs dim j with j + 16 of a block
// because one V byte holds both.
template <int FMT>
__device__ __forceinline__ int LaneDim(int lane, int k, int dpl) {
  if (FMT == 8) return lane * dpl + k;
  const int pair = lane * (dpl / 2) + k / 2;
  return (pair / 16) * 32 + pair % 16 + 16 * (k & 1);
}

// One workgroup per (split, kv head, sequence); wave w takes tiles split * tps + w, + 4, ... A lane owns one token for
// the scores and D / 64 dims for P.V. G query heads share every K and V byte read.
template <int FMT, int D>
__global__ __launch_bounds__(256) void DattnPartScalar(const DecodeArgs a) {
  constexpr int NB = D / 32, DPL = D / 64, CB = FMT == 8 ? 32 : 16;
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv, PT = g.pt;
  const int s = blockIdx.z, h = blockIdx.y, split = blockIdx.x;
  const int len = min(max(a.seq_len[s], 0), a.max_len);
  const int n_tiles = (len + kTile - 1) / kTile;
  const int tile0 = split * a.tiles_per_split;
  if (tile0 >= n_tiles) return;
  const int tile1 = min(tile0 + a.tiles_per_split, n_tiles);
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;

  __shared__ float qs[kMaxGroup][D];
  __shared__ float ps[kWaves][kMaxGroup][kTile];
  __shared__ float wm[kWaves][kMaxGroup], wl[kWaves][kMaxGroup];
  __shared__ float wacc[kWaves][kMaxGroup][D];

  for (int i = threadIdx.x; i < G * D; i += 256)
    qs[i / D][i % D] = LoadSrc(a.q, (size_t(s) * g.n_q + size_t(h) * G) * D + i, a.q_dtype);
  __syncthreads();

  float m[kMaxGroup], l[kMaxGroup], acc[kMaxGroup][DPL];
#pragma unroll
  for (int gi = 0; gi < kMaxGroup; ++gi) {
    m[gi] = kNegMax, l[gi] = 0.0f;
#pragma unroll
    for (int k = 0; k < DPL; ++k) acc[gi][k] = 0.0f;
  }
  const int32_t* row = a.table + int64_t(s) * a.stride;

  for (int tile = tile0 + wave; tile < tile1; tile += kWaves) {
    // ---- scores: lane = token
    const int tok = tile * kTile + lane;
    const bool valid = tok < len;
    float sc[kMaxGroup];
#pragma unroll
    for (int gi = 0; gi < kMaxGroup; ++gi) sc[gi] = 0.0f;
    if (valid) {
      const size_t ph = size_t(ClampPage(row[tok / PT], g.n_pages)) * H + h;
      const int t = tok % PT;
      for (int b = 0; b < NB; ++b) {
        const float d = WidenF16(a.pools.ks[(ph * PT + t) * NB + b]);
        const uint4* cp = reinterpret_cast<const uint4*>(a.pools.kq + ((ph * NB + b) * PT + t) * CB);
        float part[kMaxGroup];
#pragma unroll
        for (int gi = 0; gi < kMaxGroup; ++gi) part[gi] = 0.0f;
#pragma unroll
        for (int c = 0; c < CB / 16; ++c) {
          const uint4 v = cp[c];
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int j = 0; j < 16; ++j) {
            const uint32_t byte = (w[j / 4] >> (8 * (j % 4))) & 0xFF;
            if (FMT == 8) {
              const float x = static_cast<float>(static_cast<int8_t>(byte));
#pragma unroll
              for (int gi = 0; gi < kMaxGroup; ++gi)
                if (gi < G) part[gi] = __builtin_fmaf(qs[gi][b * 32 + c * 16 + j], x, part[gi]);
            } else {
              const float x0 = static_cast<float>(int(byte & 0xF) - 8), x1 = static_cast<float>(int(byte >> 4) - 8);
#pragma unroll
              for (int gi = 0; gi < kMaxGroup; ++gi)
                if (gi < G) {
                  part[gi] = __builtin_fmaf(qs[gi][b * 32 + j], x0, part[gi]);
                  part[gi] = __builtin_fmaf(qs[gi][b * 32 + 16 + j], x1, part[gi]);
                }
            }
          }
        }
#pragma unroll
        for (int gi = 0; gi < kMaxGroup; ++gi) sc[gi] = __builtin_fmaf(d, part[gi], sc[gi]);
      }
    }
    // ---- online softmax per head, across the wave's 64 tokens
#pragma unroll
    for (int gi = 0; gi < kMaxGroup; ++gi) {
      if (gi < G) {
        const float sv = valid ? sc[gi] * a.scale : kNegMax;
        const float mn = fmaxf(m[gi], WaveMax(sv));
        const float alpha = __expf(m[gi] - mn);
        const float p = valid ? __expf(sv - mn) : 0.0f;
        l[gi] = l[gi] * alpha + WaveSum(p);
#pragma unroll
        for (int k = 0; k < DPL; ++k) acc[gi][k] *= alpha;
        m[gi] = mn;
        ps[wave][gi][lane] = p;
      }
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- P.V: lane = D / 64 dims, loop over the tile's pages and tokens
    for (int sp = 0; sp < kTile / PT; ++sp) {
      const int base = tile * kTile + sp * PT;
      if (base >= len) break;
      const int nt = min(PT, len - base);
      const size_t ph = size_t(ClampPage(row[base / PT], g.n_pages)) * H + h;
#pragma unroll
      for (int k = 0; k < DPL; k += (FMT == 8 ? 1 : 2)) {
        const int d0 = LaneDim<FMT>(lane, k, DPL);
        const int b = d0 / 32;
        const uint16_t* sp16 = a.pools.vs + (ph * NB + b) * PT;
        const uint8_t* cp = FMT == 8 ? a.pools.vq + (ph * D + d0) * PT
                                     : a.pools.vq + ((ph * NB + b) * 16 + d0 % 32) * PT;
        for (int t = 0; t < nt; ++t) {
          const float d = WidenF16(sp16[t]);
          const uint32_t byte = cp[t];
          if (FMT == 8) {
            const float v = d * static_cast<float>(static_cast<int8_t>(byte));
#pragma unroll
            for (int gi = 0; gi < kMaxGroup; ++gi)
              if (gi < G) acc[gi][k] = __builtin_fmaf(ps[wave][gi][sp * PT + t], v, acc[gi][k]);
          } else {
            const float v0 = d * static_cast<float>(int(byte & 0xF) - 8), v1 = d * static_cast<float>(int(byte >> 4) - 8);
#pragma unroll
            for (int gi = 0; gi < kMaxGroup; ++gi)
              if (gi < G) {
                const float p = ps[wave][gi][sp * PT + t];
                acc[gi][k] = __builtin_fmaf(p, v0, acc[gi][k]);
                acc[gi][k + 1] = __builtin_fmaf(p, v1, acc[gi][k + 1]);
              }
          }
        }
      }
    }
    __builtin_amdgcn_wave_barrier();  // ps is rewritten by the next tile
  }

  // ---- merge the four waves, write the split's partial
#pragma unroll
  for (int gi = 0; gi < kMaxGroup; ++gi) {
    if (gi < G) {
      if (lane == 0) wm[wave][gi] = m[gi], wl[wave][gi] = l[gi];
#pragma unroll
      for (int k = 0; k < DPL; ++k) wacc[wave][gi][LaneDim<FMT>(lane, k, DPL)] = acc[gi][k];
    }
  }
  __syncthreads();
  const size_t part = ((size_t(s) * H + h) * a.n_splits + split) * G;
  for (int i = threadIdx.x; i < G * D; i += 256) {
    const int gi = i / D, d = i % D;
    float M = kNegMax;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) M = fmaxf(M, wm[w][gi]);
    float L = 0.0f, A = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float e = __expf(wm[w][gi] - M);
      L = __builtin_fmaf(e, wl[w][gi], L);
      A = __builtin_fmaf(e, wacc[w][gi][d], A);
    }
    a.acc[(part + gi) * D + d] = A;
    if (d == 0) a.ml[(part + gi) * 2] = M, a.ml[(part + gi) * 2 + 1] = L;
  }
}

// ---- q8_0 on the matrix cores -----------------------------------------------------------------------------------------
//
// A scalar-ALU version of this kernel needs 7 lane operations per KV byte (one convert and one multiply-add per query
// head of the group): at 5.6 TB/s that is every VALU issue slot of the chip. So the two contractions go to MFMA, whose
// f16 rate leaves both at a few percent of peak, and the VALU only converts codes (about 1.5 operations per byte):
//   scores  S[head][token] = sum_block ks[token][block] * (Q_block . codes_block)   v_mfma_f32_32x32x16_f16, one
//           32-dim block per pair of instructions (K = 16 each), so the block scale is applied to the f32 result and
//           the products themselves are exact (int8 codes and f16 queries are exact in f16)
//   output  O[head][dim] += sum_token P[head][token] * (vs[token][block] * codes)   v_mfma_f32_16x16x32_f16; the scale
//           varies along the contraction here, so V is dequantized to f16 (one rounding, 2^-12 relative)
// The page layouts are chosen for these operand shapes: a lane's 16-byte load is 16 dims of one key (K, [block][token]
// [32]) or 16 keys of one dim (V^T, [dim][token]); each wave-wide load is 1 KB contiguous.
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef _Float16 h8v __attribute__((ext_vector_type(8)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

// Eight int8 codes (two dwords) as eight f16, exact. 0x6400 | u is the f16 1024 + u; u = code + 128.
__device__ __forceinline__ h8v Codes8(uint32_t w0, uint32_t w1) {
  const h2v off = {static_cast<_Float16>(-1152.0f), static_cast<_Float16>(-1152.0f)};
  const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
  const h2v a = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u)) + off;
  const h2v b = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u)) + off;
  const h2v c = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u)) + off;
  const h2v d = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u)) + off;
  return h8v{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// Eight consecutive query elements as f16 (bf16 and f16 sources convert exactly in the normal f16 range).
__device__ __forceinline__ h8v LoadQ8(const void* q, size_t i, int dt) {
  h8v r;
  if (dt == YAHKV_F32) {
    const float4 a = *reinterpret_cast<const float4*>(static_cast<const float*>(q) + i);
    const float4 b = *reinterpret_cast<const float4*>(static_cast<const float*>(q) + i + 4);
    const float v[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = static_cast<_Float16>(v[j]);
  } else {
    const uint4 a = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(q) + i);
    const uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint16_t hbits = static_cast<uint16_t>(w[j / 2] >> (16 * (j % 2)));
      r[j] = dt == YAHKV_F16 ? __builtin_bit_cast(_Float16, hbits) : static_cast<_Float16>(WidenBf16(hbits));
    }
  }
  return r;
}

__device__ __forceinline__ float HalfMax32(float v) {  // over the 32 lanes of a wave half
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float HalfSum32(float v) {
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

// One workgroup per (split, kv head, sequence), four waves, each with its own tiles of 64 keys and its own online
// softmax; merged through LDS at the end. Loads run one tile ahead of the arithmetic: V of the tile is in flight while
// its scores are computed, K of the wave's next tile while P.V is. Page numbers come through scalar loads (they are
// the same for the whole wave), so waiting for them does not drain the vector-memory queue.
template <int D, int PT>
__global__ __launch_bounds__(256) void DattnPartQ8(const DecodeArgs a) {
  constexpr int NB = D / 32, NT = D / 16, PPT = kTile / PT;
  constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const int s = blockIdx.z, h = blockIdx.y, split = blockIdx.x;
  const int len = min(max(a.seq_len[s], 0), a.max_len);
  const int n_tiles = (len + kTile - 1) / kTile;
  const int tile0 = split * a.tiles_per_split;
  if (tile0 >= n_tiles) return;
  const int tile1 = min(tile0 + a.tiles_per_split, n_tiles);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
  const int n32 = lane % 32, half = lane / 32;  // score layout: lane = key (mod 32), registers = heads 4 * half + r
  const int n16 = lane % 16, kg = lane / 16;    // P.V layout: lane = dim (mod 16), 16 keys per lane group

  __shared__ __align__(16) _Float16 lq[NB][2][64][8];  // query A-operands, [block][K half][lane]
  __shared__ __align__(16) _Float16 lp[kWaves][kMaxGroup][kTile];
  __shared__ __align__(16) _Float16 lvs[kWaves][NB][kTile];
  __shared__ float wm[kWaves][kMaxGroup], wl[kWaves][kMaxGroup];
  __shared__ float wacc[kWaves][kMaxGroup][D];

  // Query operands: row m of the 32-row A matrix is head m of the group (rows past G are zero); lane (m, half) holds
  // dims 32 b + 16 half + 8 sub + 0..7 for the (b, sub) instruction, matching the 16 code bytes a key lane loads.
  for (int i = threadIdx.x; i < NB * 2 * 64; i += 256) {
    const int b = i / 128, sub = (i / 64) % 2, l = i % 64;
    h8v v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (l % 32 < G)
      v = LoadQ8(a.q, (size_t(s) * g.n_q + size_t(h) * G + l % 32) * D + b * 32 + 16 * (l / 32) + 8 * sub, a.q_dtype);
    *reinterpret_cast<h8v*>(&lq[b][sub][l][0]) = v;
  }
  __syncthreads();

  const int32_t* row = a.table + int64_t(s) * a.stride;
  // (page, kv head) index of the key `tok_in_tile` of a tile; page numbers are wave-uniform loads.
  auto page_head = [&](const int (&pg)[PPT], int tok_in_tile) -> size_t {
    int p = pg[0];
#pragma unroll
    for (int j = 1; j < PPT; ++j) p = tok_in_tile / PT == j ? pg[j] : p;
    return size_t(p) * H + h;
  };
  auto load_pages = [&](int tile, int (&pg)[PPT]) {
#pragma unroll
    for (int j = 0; j < PPT; ++j) pg[j] = ClampPage(row[min(tile * PPT + j, a.stride - 1)], g.n_pages);
  };

  uint4 kb[NB][2];   // [block][32-key half of the tile]: 16 codes of this lane's key
  uint4 ksc[2];      // the key's NB block scales (f16)
  uint4 vb[NT];      // [16-dim tile]: 16 keys of this lane's dim
  uint4 vsr;         // staging of the tile's V scales: 8 keys of one block per lane
  auto load_k = [&](const int (&pg)[PPT]) {
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const int tk = 32 * tt + n32;
      const size_t ph = page_head(pg, tk);
      const int t = tk % PT;
#pragma unroll
      for (int b = 0; b < NB; ++b)
        kb[b][tt] = *reinterpret_cast<const uint4*>(a.pools.kq + ((ph * NB + b) * PT + t) * 32 + 16 * half);
      const uint16_t* sp = a.pools.ks + (ph * PT + t) * NB;
      if (NB == 8) {
        ksc[tt] = *reinterpret_cast<const uint4*>(sp);
      } else {
        const uint2 v = *reinterpret_cast<const uint2*>(sp);
        ksc[tt] = uint4{v.x, v.y, 0u, 0u};
      }
    }
  };
  auto load_v = [&](const int (&pg)[PPT]) {
    const size_t ph = page_head(pg, 16 * kg);
    const int t0 = (16 * kg) % PT;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      vb[nt] = *reinterpret_cast<const uint4*>(a.pools.vq + (ph * D + 16 * nt + n16) * PT + t0);
    const int b = lane / 8, chunk = lane % 8;  // V scales: lane = (block, 8 keys)
    if (b < NB) {
      const size_t ps = page_head(pg, 8 * chunk);
      vsr = *reinterpret_cast<const uint4*>(a.pools.vs + (ps * NB + b) * PT + (8 * chunk) % PT);
    }
  };

  float m[4], lsum[4];
  f4v o[NT];
#pragma unroll
  for (int r = 0; r < 4; ++r) m[r] = kNegMax, lsum[r] = 0.0f;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) o[nt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
  const float qk_scale = a.scale * kLog2e;  // softmax in base 2
  // P rows read back as A-matrix rows: rows 0-3 are heads 0-3, rows 8-11 heads 4-7, so that a lane's output rows are
  // the heads whose running maximum it already holds (lanes 0-15: heads 0-3, lanes 32-47: heads 4-7).
  const int prow = n16 < 4 ? n16 : (n16 >= 8 && n16 < 12 ? n16 - 4 : 0);

  int tile = tile0 + wave;
  int pg[PPT];
  if (tile < tile1) {
    load_pages(tile, pg);
    load_k(pg);
    load_v(pg);
  }
  for (; tile < tile1; tile += kWaves) {
    const int next = tile + kWaves;
    if (next < tile1) load_pages(next, pg);
    // ---- scores
    float sc[2][4];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int r = 0; r < 4; ++r) sc[tt][r] = 0.0f;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const h8v q0 = *reinterpret_cast<const h8v*>(&lq[b][0][lane][0]);
      const h8v q1 = *reinterpret_cast<const h8v*>(&lq[b][1][lane][0]);
      f16v c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0;
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(q0, Codes8(kb[b][0].x, kb[b][0].y), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(q0, Codes8(kb[b][1].x, kb[b][1].y), c1, 0, 0, 0);
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(q1, Codes8(kb[b][0].z, kb[b][0].w), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(q1, Codes8(kb[b][1].z, kb[b][1].w), c1, 0, 0, 0);
      const uint32_t w0 = b < 2 ? ksc[0].x : b < 4 ? ksc[0].y : b < 6 ? ksc[0].z : ksc[0].w;
      const uint32_t w1 = b < 2 ? ksc[1].x : b < 4 ? ksc[1].y : b < 6 ? ksc[1].z : ksc[1].w;
      const float d0 = WidenF16(static_cast<uint16_t>(w0 >> (16 * (b % 2)))) * qk_scale;
      const float d1 = WidenF16(static_cast<uint16_t>(w1 >> (16 * (b % 2)))) * qk_scale;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        sc[0][r] = __builtin_fmaf(c0[r], d0, sc[0][r]);
        sc[1][r] = __builtin_fmaf(c1[r], d1, sc[1][r]);
      }
      // One block (two independent accumulator chains) at a time: more only multiplies live 32x32 accumulators.
      // The empty asm pins the scaled sums here, so the accumulators die before the next block starts.
      asm volatile("" : "+v"(sc[0][0]), "+v"(sc[0][1]), "+v"(sc[0][2]), "+v"(sc[0][3]), "+v"(sc[1][0]), "+v"(sc[1][1]),
                        "+v"(sc[1][2]), "+v"(sc[1][3]));
      __builtin_amdgcn_sched_barrier(0);
    }
    if (next < tile1) load_k(pg);
    // ---- online softmax (base 2); keys at or past len are masked by select, so stale scales cannot leak
    float alpha[4];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const bool valid = tile * kTile + 32 * tt + n32 < len;
#pragma unroll
      for (int r = 0; r < 4; ++r) sc[tt][r] = valid ? sc[tt][r] : kNegMax;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float mn = fmaxf(m[r], HalfMax32(fmaxf(sc[0][r], sc[1][r])));
      alpha[r] = __builtin_amdgcn_exp2f(m[r] - mn);
      m[r] = mn;
      const float p0 = __builtin_amdgcn_exp2f(sc[0][r] - mn), p1 = __builtin_amdgcn_exp2f(sc[1][r] - mn);
      lsum[r] = __builtin_fmaf(lsum[r], alpha[r], p0 + p1);  // per lane; summed over the lanes at the end
      lp[wave][4 * half + r][n32] = static_cast<_Float16>(p0);
      lp[wave][4 * half + r][32 + n32] = static_cast<_Float16>(p1);
    }
    {  // V scales of the tile to LDS; scales of keys at or past len become 0, which makes their V rows 0
      const int b = lane / 8, chunk = lane % 8;
      if (b < NB) {
        uint32_t w[4] = {vsr.x, vsr.y, vsr.z, vsr.w};
        const int k0 = tile * kTile + 8 * chunk;
        if (k0 + 8 > len) {
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (k0 + j >= len) w[j / 2] &= j % 2 ? 0x0000FFFFu : 0xFFFF0000u;
        }
        *reinterpret_cast<uint4*>(&lvs[wave][b][8 * chunk]) = uint4{w[0], w[1], w[2], w[3]};
      }
    }
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[nt][r] *= alpha[r];
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    // ---- P.V
    const h8v pa0 = *reinterpret_cast<const h8v*>(&lp[wave][prow][16 * kg]);
    const h8v pa1 = *reinterpret_cast<const h8v*>(&lp[wave][prow][16 * kg + 8]);
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const h8v s0 = *reinterpret_cast<const h8v*>(&lvs[wave][b][16 * kg]);
      const h8v s1 = *reinterpret_cast<const h8v*>(&lvs[wave][b][16 * kg + 8]);
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int nt = 2 * b + j;
        const h8v v0 = Codes8(vb[nt].x, vb[nt].y) * s0, v1 = Codes8(vb[nt].z, vb[nt].w) * s1;
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa0, v0, o[nt], 0, 0, 0);
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa1, v1, o[nt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_wave_barrier();  // lp / lvs are rewritten by the next tile
    if (next < tile1) load_v(pg);
  }

  // ---- merge the four waves (natural-log units, as the reduce expects), write the split's partial
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float l = HalfSum32(lsum[r]);
    if (n32 == 0) wm[wave][4 * half + r] = m[r] * kLn2, wl[wave][4 * half + r] = l;
  }
  if (kg == 0 || kg == 2) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) wacc[wave][2 * kg + r][16 * nt + n16] = o[nt][r];
  }
  __syncthreads();
  const size_t part = ((size_t(s) * H + h) * a.n_splits + split) * G;
  for (int i = threadIdx.x; i < G * D; i += 256) {
    const int gi = i / D, d = i % D;
    float M = kNegMax;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) M = fmaxf(M, wm[w][gi]);
    float L = 0.0f, A = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float e = __expf(wm[w][gi] - M);
      L = __builtin_fmaf(e, wl[w][gi], L);
      A = __builtin_fmaf(e, wacc[w][gi][d], A);
    }
    a.acc[(part + gi) * D + d] = A;
    if (d == 0) a.ml[(part + gi) * 2] = M, a.ml[(part + gi) * 2 + 1] = L;
  }
}

// One workgroup per (query head, sequence), thread = dim (gen_decode_attn.py:338-411).
__global__ void DattnReduce(const DecodeArgs a) {
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv, D = g.hd;
  const int hq = blockIdx.x, s = blockIdx.y, d = threadIdx.x;
  const int h = hq / G, gi = hq % G;
  const int len = min(max(a.seq_len[s], 0), a.max_len);
  const size_t o = (size_t(s) * g.n_q + hq) * D + d;
  if (len == 0) {
    a.out[o] = 0.0f;
    return;
  }
  const int n_tiles = (len + kTile - 1) / kTile;
  const int ns = (n_tiles + a.tiles_per_split - 1) / a.tiles_per_split;
  const size_t part = (size_t(s) * H + h) * a.n_splits * G + gi;
  float M = kNegMax;
  for (int sp = 0; sp < ns; ++sp) M = fmaxf(M, a.ml[(part + size_t(sp) * G) * 2]);
  float L = 0.0f, A = 0.0f;
  for (int sp = 0; sp < ns; ++sp) {
    const size_t p = part + size_t(sp) * G;
    const float w = __expf(a.ml[p * 2] - M);
    L = __builtin_fmaf(w, a.ml[p * 2 + 1], L);
    A = __builtin_fmaf(w, a.acc[p * D + d], A);
  }
  float v = A / L;
  if (a.gate != nullptr) v *= 1.0f / (1.0f + __expf(-a.gate[o]));
  a.out[o] = v;
}

// Slices of the context: enough workgroups to fill 256 CUs several times over, at least one tile per wave.
struct Plan {
  int32_t max_len, n_splits, tiles_per_split;
};
Plan MakePlan(const Geom& g, int32_t n_seqs, int32_t max_seq_len) {
  Plan p;
  p.max_len = std::max(max_seq_len, 1);
  const int64_t max_tiles = (int64_t(p.max_len) + kTile - 1) / kTile;
  const int64_t want_wgs = 2048;
  int64_t tps = (max_tiles * g.n_kv * n_seqs + want_wgs - 1) / want_wgs;
  tps = std::max<int64_t>(tps, kWaves);
  tps = (tps + kWaves - 1) / kWaves * kWaves;
  p.tiles_per_split = static_cast<int32_t>(tps);
  p.n_splits = static_cast<int32_t>((max_tiles + tps - 1) / tps);
  return p;
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" size_t yahkv_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len) {
  if (CheckGeometry(g) || n_seqs <= 0 || max_seq_len <= 0) return 0;
  const Geom m = MakeGeom(*g);
  const Plan p = MakePlan(m, n_seqs, max_seq_len);
  return size_t(n_seqs) * m.n_kv * p.n_splits * m.group() * (m.hd + 2) * sizeof(float);
}

namespace {

// Fills the launch arguments both dispatches share; returns a status.
int Prepare(const yahkv_geometry* g, int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
            int32_t max_seq_len, const void* workspace, size_t workspace_bytes, DecodeArgs* a) {
  if (const int st = CheckGeometry(g)) return st;
  if (seq_len == nullptr || workspace == nullptr) return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || max_seq_len <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (reinterpret_cast<uintptr_t>(workspace) & 15) return YAHKV_ERR_ARG;
  if (workspace_bytes < yahkv_decode_workspace_bytes(g, n_seqs, max_seq_len)) return YAHKV_ERR_WORKSPACE;
  const Geom m = MakeGeom(*g);
  const Plan p = MakePlan(m, n_seqs, max_seq_len);
  *a = DecodeArgs{};
  a->g = m, a->stride = page_table_stride, a->seq_len = seq_len, a->n_seqs = n_seqs;
  // lengths read on the device are clamped to the host's bound and to the table's extent
  a->max_len = static_cast<int32_t>(std::min<int64_t>(p.max_len, int64_t(page_table_stride) * m.pt));
  a->acc = static_cast<float*>(const_cast<void*>(workspace));
  a->ml = a->acc + size_t(n_seqs) * m.n_kv * p.n_splits * m.group() * m.hd;
  a->n_splits = p.n_splits, a->tiles_per_split = p.tiles_per_split;
  return YAHKV_OK;
}

}  // namespace

extern "C" int yahkv_decode_part(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                 int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                 int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                 void* workspace, size_t workspace_bytes, void* stream) {
  DecodeArgs a;
  if (const int st = Prepare(g, page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, &a))
    return st;
  if (pools == nullptr || pools->kq == nullptr || pools->ks == nullptr || pools->vq == nullptr ||
      pools->vs == nullptr || page_table == nullptr || q == nullptr)
    return YAHKV_ERR_ARG;
  if (q_dtype != YAHKV_F32 && q_dtype != YAHKV_F16 && q_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(pools->kq) | reinterpret_cast<uintptr_t>(pools->vq) |
       reinterpret_cast<uintptr_t>(pools->ks) | reinterpret_cast<uintptr_t>(pools->vs)) & 15)
    return YAHKV_ERR_ARG;
  a.pools = MakePools(*pools), a.table = page_table, a.q = q, a.q_dtype = q_dtype, a.scale = softmax_scale;
  const Geom& m = a.g;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(a.n_splits, m.n_kv, n_seqs);
  if (m.format == 8) {
#define YAHKV_LAUNCH_Q8(DD, PP) hipLaunchKernelGGL((DattnPartQ8<DD, PP>), grid, dim3(256), 0, st, a)
    if (m.hd == 256 && m.pt == 64) YAHKV_LAUNCH_Q8(256, 64);
    else if (m.hd == 256 && m.pt == 32) YAHKV_LAUNCH_Q8(256, 32);
    else if (m.hd == 256) YAHKV_LAUNCH_Q8(256, 16);
    else if (m.pt == 64) YAHKV_LAUNCH_Q8(128, 64);
    else if (m.pt == 32) YAHKV_LAUNCH_Q8(128, 32);
    else YAHKV_LAUNCH_Q8(128, 16);
#undef YAHKV_LAUNCH_Q8
  } else if (m.hd == 256) {
    hipLaunchKernelGGL((DattnPartScalar<4, 256>), grid, dim3(256), 0, st, a);
  } else {
    hipLaunchKernelGGL((DattnPartScalar<4, 128>), grid, dim3(256), 0, st, a);
  }
  return LaunchStatus();
}

extern "C" int yahkv_decode_reduce(const yahkv_geometry* g, int32_t page_table_stride, const int32_t* seq_len,
                                   int32_t n_seqs, int32_t max_seq_len, const float* gate, float* out,
                                   const void* workspace, size_t workspace_bytes, void* stream) {
  DecodeArgs a;
  if (const int st = Prepare(g, page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, &a))
    return st;
  if (out == nullptr) return YAHKV_ERR_ARG;
  a.gate = gate, a.out = out;
  hipLaunchKernelGGL(DattnReduce, dim3(a.g.n_q, n_seqs), dim3(a.g.hd), 0, static_cast<hipStream_t>(stream), a);
  return LaunchStatus();
}

extern "C" int yahkv_decode_attend(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                   int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                   int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                   const float* gate, float* out, void* workspace, size_t workspace_bytes,
                                   void* stream) {
  if (out == nullptr) return YAHKV_ERR_ARG;
  if (const int st = yahkv_decode_part(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q,
                                       q_dtype, softmax_scale, workspace, workspace_bytes, stream))
    return st;
  return yahkv_decode_reduce(g, page_table_stride, seq_len, n_seqs, max_seq_len, gate, out, workspace,
                             workspace_bytes, stream);
}
