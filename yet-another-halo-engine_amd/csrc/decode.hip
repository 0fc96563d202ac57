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
__global__ __launch_bounds__(256) void DattnPart(const DecodeArgs a) {
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
  if (m.format == 8 && m.hd == 256) hipLaunchKernelGGL((DattnPart<8, 256>), grid, dim3(256), 0, st, a);
  else if (m.format == 8) hipLaunchKernelGGL((DattnPart<8, 128>), grid, dim3(256), 0, st, a);
  else if (m.hd == 256) hipLaunchKernelGGL((DattnPart<4, 256>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((DattnPart<4, 128>), grid, dim3(256), 0, st, a);
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
