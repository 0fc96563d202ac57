// Append fused with head RMSNorm and NeoX RoPE: K rows are normalised and rotated in registers / LDS and go straight
// into their quantized page; V rows are quantized as they are; Q rows, if given, are normalised and rotated on the way.
//
// Follows the reference's fused decode kernel (engine/gpu/loom/yah_fused_qk_rope_f32.loom:1-10, Q branch :96-146,
// K branch :147-241) and its batched, paged rewrite for prefill chunks (engine/gpu/loom/tools/emit_prefill_pp.py:
// 31-111): per head
//   inv_rms = rsqrt(sum_i x[i]^2 / head_dim + eps); normed[i] = (x[i] * inv_rms) * weight[i]
//   angle(p) = pos * (1 / theta^(2 p / rotary_dim)), p < half = rotary_dim / 2
//   out[p] = normed[p] cos - normed[p + half] sin; out[p + half] = normed[p] sin + normed[p + half] cos
// and dims at or past rotary_dim are only normalised. The angle uses the token's position as given; the page slot
// uses the position clamped to the table, as in the reference (:89-94).
// What the reference stores as f16 rows is stored here as q8_0 / q4_0 blocks: this removes the f32 round trip of the
// rotated K through memory between the rotation and the quantizer.
#include <type_traits>

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
};

// Four consecutive elements of a source / destination row (element index a multiple of 4).
__device__ __forceinline__ float4 Load4(const void* src, size_t i, int dtype) {
  if (dtype == YAHKV_F32) return *reinterpret_cast<const float4*>(static_cast<const float*>(src) + i);
  const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(src) + i);
  const uint16_t h[4] = {static_cast<uint16_t>(w.x & 0xFFFF), static_cast<uint16_t>(w.x >> 16),
                         static_cast<uint16_t>(w.y & 0xFFFF), static_cast<uint16_t>(w.y >> 16)};
  if (dtype == YAHKV_F16) return float4{WidenF16(h[0]), WidenF16(h[1]), WidenF16(h[2]), WidenF16(h[3])};
  return float4{WidenBf16(h[0]), WidenBf16(h[1]), WidenBf16(h[2]), WidenBf16(h[3])};
}
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

template <int CTRL>
__device__ __forceinline__ float Dpp(float x) {  // the value of another lane of the row, chosen by a DPP control
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int DppI(int x) { return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xF, 0xF, false); }
constexpr int kQuadSwap1 = 0xB1, kQuadSwap2 = 0x4E, kHalfMirror = 0x141, kRowMirror = 0x140;

// Sum over the 64 lanes, in every lane: four DPP steps inside each row of 16 lanes, then the two row-swapping
// instructions of gfx950 across the rows (no LDS round trips).
__device__ __forceinline__ float WaveSum(float v) {
  v += Dpp<kQuadSwap1>(v);
  v += Dpp<kQuadSwap2>(v);
  v += Dpp<kHalfMirror>(v);
  v += Dpp<kRowMirror>(v);
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const uint32_t r0 = r[0], r1 = r[1];
  const float w = __builtin_bit_cast(float, r0) + __builtin_bit_cast(float, r1);
  const uint32_t x = __builtin_bit_cast(uint32_t, w);
  const auto q = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  const uint32_t q0 = q[0], q1 = q[1];
  return __builtin_bit_cast(float, q0) + __builtin_bit_cast(float, q1);
}

// A block of 32 values lies in 8 consecutive lanes, 4 values each (lane l of the 8: elements 4 l .. 4 l + 3).
// q8_0: the block's amax in all 8 lanes (a maximum does not depend on the order), then the scalar formulas of
// QuantizeBlock per element; returns this lane's 4 codes packed into a dword.
__device__ __forceinline__ uint32_t QuantizeLanesQ8(const float4 v, uint16_t* scale) {
#pragma clang fp contract(off)
  float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
  amax = fmaxf(amax, Dpp<kQuadSwap1>(amax));
  amax = fmaxf(amax, Dpp<kQuadSwap2>(amax));
  amax = fmaxf(amax, Dpp<kHalfMirror>(amax));
  const float d = amax / 127.0f;
  const float inv = d > 0.0f ? 1.0f / d : 0.0f;
  *scale = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d));
  const uint32_t c0 = static_cast<uint8_t>(static_cast<int8_t>(CodeQ8(v.x * inv)));
  const uint32_t c1 = static_cast<uint8_t>(static_cast<int8_t>(CodeQ8(v.y * inv)));
  const uint32_t c2 = static_cast<uint8_t>(static_cast<int8_t>(CodeQ8(v.z * inv)));
  const uint32_t c3 = static_cast<uint8_t>(static_cast<int8_t>(CodeQ8(v.w * inv)));
  return c0 | (c1 << 8) | (c2 << 16) | (c3 << 24);
}
// q4_0: ggml takes the value of largest magnitude, the first one on ties, so the reduction carries (|x|, index,
// x) and prefers the lower index; d = that value / -8. Lanes 0-3 of the 8 return 4 bytes: low nibbles their own
// elements j, high nibbles the elements j + 16 held by the lane four further on.
__device__ __forceinline__ uint32_t QuantizeLanesQ4(const float4 v, int lane_in_block, uint16_t* scale) {
#pragma clang fp contract(off)
  const float e[4] = {v.x, v.y, v.z, v.w};
  float av = fabsf(e[0]), mx = e[0];
  int ix = 4 * lane_in_block;
#pragma unroll
  for (int j = 1; j < 4; ++j)
    if (av < fabsf(e[j])) av = fabsf(e[j]), mx = e[j], ix = 4 * lane_in_block + j;
  auto merge = [&](float oav, float omx, int oix) {
    if (oav > av || (oav == av && oix < ix)) av = oav, mx = omx, ix = oix;
  };
  merge(Dpp<kQuadSwap1>(av), Dpp<kQuadSwap1>(mx), DppI<kQuadSwap1>(ix));
  merge(Dpp<kQuadSwap2>(av), Dpp<kQuadSwap2>(mx), DppI<kQuadSwap2>(ix));
  merge(Dpp<kHalfMirror>(av), Dpp<kHalfMirror>(mx), DppI<kHalfMirror>(ix));
  const float d = mx / -8.0f;
  const float id = d != 0.0f ? 1.0f / d : 0.0f;
  *scale = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d));
  uint32_t nib = 0;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int q = min(15, static_cast<int>(static_cast<int8_t>(static_cast<int>(e[j] * id + 8.5f))));
    nib |= static_cast<uint32_t>(q) << (8 * j);
  }
  // the nibbles of the lane four further on (row_shr would move the wrong way: take them through a lane shuffle)
  const uint32_t hi = static_cast<uint32_t>(__shfl_down(static_cast<int>(nib), 4, 64));
  return nib | (hi << 4);
}

// One workgroup of four wavefronts per token. The token's angles (they depend on the position and the pair, not on
// the head) are computed once into LDS. The token's rows of head_dim values (its H K heads, its H V heads, then its
// query heads) are dealt to the wavefronts in turn; a row lies across a wavefront, four consecutive dims per lane, so
// every load and store is 16 (or 8) bytes per lane, the sum of squares and the block maxima are DPP reductions, and
// the partner of a rotated pair comes through one lane shuffle: rows never go through LDS. A wavefront issues the
// loads of all its rows (up to eight at a time) before it works on the first.
constexpr int kRopeWaves = 4, kRowsInFlight = 8;
template <int FMT>
__global__ __launch_bounds__(64 * kRopeWaves) void AppendRope(const RopeArgs a) {
#pragma clang fp contract(off)
  const Geom g = a.g;
  const int NB = g.nb(), H = g.n_kv, PT = g.pt, D = g.hd, NQ = a.q_src != nullptr ? g.n_q : 0;
  const int rows_per_token = 2 * H + NQ;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int i = int(blockIdx.x % a.n_new), s = int(blockIdx.x / a.n_new);
  if (a.n_valid != nullptr && i >= a.n_valid[s]) return;  // padding row of a short chunk
  const int pos_raw = a.start_pos[s] + i;
  const int pos = min(max(pos_raw, 0), a.stride * PT - 1);
  const int page = ClampPage(a.table[int64_t(s) * a.stride + pos / PT], g.n_pages);
  const int t = pos % PT;

  __shared__ __align__(16) float cs[128], sn[128];  // rotary_dim / 2 <= 128
  const int rot = a.rotary_dim, half = rot / 2;
  const float posf = static_cast<float>(pos_raw);
  for (int p = threadIdx.x; p < half; p += 64 * kRopeWaves) {
    const float inv_freq = 1.0f / powf(a.theta, (2.0f * static_cast<float>(p)) / static_cast<float>(rot));
    float sv, cv;
    sincosf(posf * inv_freq, &sv, &cv);
    cs[p] = cv, sn[p] = sv;
  }
  __syncthreads();
  const int d0 = 4 * lane;  // this lane's four dims of every row
  const bool has = d0 < D;
  // This lane's part of the rotation, the same for every row: element e = d0 + j is the first of its pair
  // (e < half: out = x c - partner s, partner = e + half), the second (half <= e < rot: out = partner s + x c,
  // partner = e - half) or past the rotated dims. rotary_dim / 2 is a multiple of 4 (checked by the entry point), so
  // the four partners lie in one lane.
  float c4[4] = {1.0f, 1.0f, 1.0f, 1.0f}, s4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
  int partner_lane = lane;
  if (has && d0 < rot) {
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
  if (a.k_weight != nullptr && has) wk = *reinterpret_cast<const float4*>(a.k_weight + d0);
  if (a.q_weight != nullptr && has) wq = *reinterpret_cast<const float4*>(a.q_weight + d0);
  // source of row `row` of the token and its element offset
  auto source = [&](int row, const void** src, size_t* off) {
    const size_t tok = size_t(s) * a.n_new + i;
    if (row < H) *src = a.k_src, *off = (tok * H + row) * D;
    else if (row < 2 * H) *src = a.v_src, *off = (tok * H + (row - H)) * D;
    else *src = a.q_src, *off = (tok * g.n_q + (row - 2 * H)) * D;
  };
  for (int first_row = wave; first_row < rows_per_token; first_row += kRopeWaves * kRowsInFlight) {
    float4 x[kRowsInFlight];
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
      const int row = first_row + kRopeWaves * j;
      x[j] = float4{0.0f, 0.0f, 0.0f, 0.0f};
      if (row < rows_per_token && has) {
        const void* src;
        size_t off;
        source(row, &src, &off);
        x[j] = Load4(src, off + d0, a.src_dtype);
      }
    }
#pragma unroll
    for (int j = 0; j < kRowsInFlight; ++j) {
      const int row = first_row + kRopeWaves * j;
      if (row >= rows_per_token) break;
      const bool is_v = row >= H && row < 2 * H, is_q = row >= 2 * H;
      float4 v = x[j];
      if (!is_v) {
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
      const int h = is_v ? row - H : row, b = lane / 8, lb = lane % 8;
      uint16_t scale;
      const uint32_t codes = FMT == 8 ? QuantizeLanesQ8(v, &scale) : QuantizeLanesQ4(v, lb, &scale);
      if (!has) continue;
      const size_t ph = size_t(page) * H + h;
      if (!is_v) {
        if (lb == 0) a.pools.ks[(ph * PT + t) * NB + b] = scale;
        if (FMT == 8)
          *reinterpret_cast<uint32_t*>(a.pools.kq + ((ph * NB + b) * PT + t) * 32 + 4 * lb) = codes;
        else if (lb < 4)
          *reinterpret_cast<uint32_t*>(a.pools.kq + ((ph * NB + b) * PT + t) * 16 + 4 * lb) = codes;
      } else {
        if (lb == 0) a.pools.vs[(ph * NB + b) * PT + t] = scale;
        if (FMT == 8) {  // row (32 b + 4 lb + e) of [D][PT]
          uint8_t* dst = a.pools.vq + (ph * D + d0) * PT + t;
#pragma unroll
          for (int e = 0; e < 4; ++e) dst[size_t(e) * PT] = static_cast<uint8_t>(codes >> (8 * e));
        } else if (lb < 4) {  // row (16 b + 4 lb + e) of [NB * 16][PT]
          uint8_t* dst = a.pools.vq + ((ph * NB + b) * 16 + 4 * lb) * PT + t;
#pragma unroll
          for (int e = 0; e < 4; ++e) dst[size_t(e) * PT] = static_cast<uint8_t>(codes >> (8 * e));
        }
      }
    }
  }
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" int yahkv_append_rope(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                 int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid,
                                 int32_t n_seqs, int32_t n_new, const void* k_src, const void* v_src,
                                 int32_t src_dtype, const yahkv_rope* rope, const void* q_src, void* q_out,
                                 int32_t q_out_dtype, float* k_out, void* stream) {
  if (const int st = CheckGeometry(g)) return st;
  if (pools == nullptr || pools->kq == nullptr || pools->ks == nullptr || pools->vq == nullptr ||
      pools->vs == nullptr || page_table == nullptr || start_pos == nullptr || k_src == nullptr ||
      v_src == nullptr || rope == nullptr)
    return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || n_new <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (src_dtype != YAHKV_F32 && src_dtype != YAHKV_F16 && src_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((q_src == nullptr) != (q_out == nullptr)) return YAHKV_ERR_ARG;
  if (q_src != nullptr && q_out_dtype != YAHKV_F32 && q_out_dtype != YAHKV_F16 && q_out_dtype != YAHKV_BF16)
    return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(pools->kq) | reinterpret_cast<uintptr_t>(pools->vq)) & 15) return YAHKV_ERR_ARG;
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
  if (g->format == YAHKV_Q8_0)
    hipLaunchKernelGGL(AppendRope<8>, dim3(static_cast<unsigned>(tokens)), dim3(64 * kRopeWaves), 0, st, a);
  else
    hipLaunchKernelGGL(AppendRope<4>, dim3(static_cast<unsigned>(tokens)), dim3(64 * kRopeWaves), 0, st, a);
  return LaunchStatus();
}
