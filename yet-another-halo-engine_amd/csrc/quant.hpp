// Block quantizers of the append kernels.
//
// Arithmetic is the reference's QuantizeQ8_0 (engine/core/gguf_quant.cpp:310-320), bit for bit: amax over the 32
// elements, d = amax / 127 (IEEE division), inv = d > 0 ? 1 / d : 0, code = lround(x * inv) (halves away from zero),
// stored scale = f16(d) (round to nearest even). q4_0 follows ggml's quantize_row_q4_0_ref. The results are compared
// bit for bit with code built with -ffp-contract=off (the reference's host flags, engine/build_hrx.sh:26), so the
// functions below forbid multiply-add fusion.
#ifndef YAHKV_QUANT_HPP_
#define YAHKV_QUANT_HPP_

#include "common.hpp"

namespace yahkv {

// A code from r = x * inv as the x86-64 reference computes it: lround. For |r| <= 128, lround(r) is the truncation of
// r + copysign(0.5 - 2^-25, r): adding the float below one half moves exactly the values with a fraction of one half
// or more past the next integer (r + 0.5 itself would also carry 0.5 - 2^-25 there, through the tie of the addition's
// rounding). Checked against lroundf for every float up to 129. Beyond that range (only reachable when 1 / d
// overflowed, i.e. amax < 2^-119: the products are then infinite or NaN) lround's result converts to the int8 0 on the
// reference's machine; CodesLanesQ8 sees to that case once per block.
__device__ __forceinline__ int RoundQ8(float r) {
#pragma clang fp contract(off)
  return static_cast<int>(r + copysignf(0x1.fffffep-2f, r));
}

template <int CTRL>
__device__ __forceinline__ float Dpp(float x) {  // the value of another lane of the row, chosen by a DPP control
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
template <int CTRL>
__device__ __forceinline__ int DppI(int x) { return __builtin_amdgcn_update_dpp(0, x, CTRL, 0xF, 0xF, false); }
constexpr int kQuadSwap1 = 0xB1, kQuadSwap2 = 0x4E, kHalfMirror = 0x141, kRowMirror = 0x140;

// The value of lane (l ^ K) of the wave, K a power of two: what `__shfl_xor(x, K, 64)` returns, without its round trip
// through LDS. Inside a row of 16 lanes DPP controls do it (l ^ 4 is a half mirror, l ^ 7, then a reversed quad,
// l ^ 3; l ^ 8 a row mirror, l ^ 15, then a half mirror); across rows the two row-swapping instructions of gfx950,
// each of which leaves the lane's own value in one result and its partner's in the other.
constexpr int kQuadReverse = 0x1B;
template <int K>
__device__ __forceinline__ uint32_t LaneXorBits(uint32_t u) {
  static_assert(K == 1 || K == 2 || K == 4 || K == 8 || K == 16 || K == 32, "one bit of the lane number");
  const int i = static_cast<int>(u);
  if constexpr (K == 1) return static_cast<uint32_t>(DppI<kQuadSwap1>(i));
  else if constexpr (K == 2) return static_cast<uint32_t>(DppI<kQuadSwap2>(i));
  else if constexpr (K == 4) return static_cast<uint32_t>(DppI<kQuadReverse>(DppI<kHalfMirror>(i)));
  else if constexpr (K == 8) return static_cast<uint32_t>(DppI<kHalfMirror>(DppI<kRowMirror>(i)));
  else if constexpr (K == 16) {
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return r0 != u ? r0 : r1;
  } else {
    const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
    const uint32_t r0 = r[0], r1 = r[1];
    return r0 != u ? r0 : r1;
  }
}
template <int K>
__device__ __forceinline__ float LaneXor(float x) {
  return __builtin_bit_cast(float, LaneXorBits<K>(__builtin_bit_cast(uint32_t, x)));
}

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
__device__ __forceinline__ float BlockAmaxQ8(const float4 v) {  // the block's amax, in all 8 lanes of the block
  float amax = fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w)));
  amax = fmaxf(amax, Dpp<kQuadSwap1>(amax));
  amax = fmaxf(amax, Dpp<kQuadSwap2>(amax));
  return fmaxf(amax, Dpp<kHalfMirror>(amax));
}
// d and 1 / d of a block from its amax, with the reference's operations
__device__ __forceinline__ void ScaleQ8(float amax, float* inv, uint16_t* scale) {
#pragma clang fp contract(off)
  const float d = amax / 127.0f;
  *inv = d > 0.0f ? 1.0f / d : 0.0f;
  *scale = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d));
}
// This lane's 4 codes in a dword. |x * inv| is at most 127 (and a bit of rounding) whenever inv is finite, so whether
// the products are in RoundQ8's range is one question per block, asked of inv.
__device__ __forceinline__ uint32_t CodesLanesQ8(const float4 v, float inv) {
#pragma clang fp contract(off)
  const uint32_t c0 = static_cast<uint32_t>(RoundQ8(v.x * inv)) & 0xFFu, c1 = static_cast<uint32_t>(RoundQ8(v.y * inv)) & 0xFFu;
  const uint32_t c2 = static_cast<uint32_t>(RoundQ8(v.z * inv)) & 0xFFu, c3 = static_cast<uint32_t>(RoundQ8(v.w * inv)) & 0xFFu;
  return inv < __builtin_inff() ? c0 | (c1 << 8) | (c2 << 16) | (c3 << 24) : 0u;
}
__device__ __forceinline__ uint32_t QuantizeLanesQ8(const float4 v, uint16_t* scale) {
  float inv;
  ScaleQ8(BlockAmaxQ8(v), &inv, scale);
  return CodesLanesQ8(v, inv);
}
// q4_0: ggml takes the value of largest magnitude, the first one on ties, so the reduction carries (|x|, index,
// x) and prefers the lower index; d = that value / -8. Lanes 0-3 of the 8 return 4 bytes: low nibbles their own
// elements j, high nibbles the elements j + 16 held by the lane four further on.
// `own`, if given, receives this lane's own four nibbles, one per byte.
__device__ __forceinline__ uint32_t QuantizeLanesQ4(const float4 v, int lane_in_block, uint16_t* scale,
                                                    uint32_t* own = nullptr) {
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
  if (own != nullptr) *own = nib;
  // the nibbles of the lane four further on (row_shr would move the wrong way: take them through a lane shuffle)
  const uint32_t hi = static_cast<uint32_t>(__shfl_down(static_cast<int>(nib), 4, 64));
  return nib | (hi << 4);
}

// Four consecutive elements of a source row of f32, f16 or bf16 values (element index a multiple of 4).
__device__ __forceinline__ float4 Load4(const void* src, size_t i, int dtype) {
  if (dtype == YAHKV_F32) return *reinterpret_cast<const float4*>(static_cast<const float*>(src) + i);
  const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(src) + i);
  const uint16_t h[4] = {static_cast<uint16_t>(w.x & 0xFFFF), static_cast<uint16_t>(w.x >> 16),
                         static_cast<uint16_t>(w.y & 0xFFFF), static_cast<uint16_t>(w.y >> 16)};
  if (dtype == YAHKV_F16) return float4{WidenF16(h[0]), WidenF16(h[1]), WidenF16(h[2]), WidenF16(h[3])};
  return float4{WidenBf16(h[0]), WidenBf16(h[1]), WidenBf16(h[2]), WidenBf16(h[3])};
}

// The same in two steps, for loads that stay in flight while other work is done: the raw bytes, widened later.
__device__ __forceinline__ uint4 LoadRaw4(const void* src, size_t i, int dtype) {
  if (dtype == YAHKV_F32) return *reinterpret_cast<const uint4*>(static_cast<const float*>(src) + i);
  const uint2 w = *reinterpret_cast<const uint2*>(static_cast<const uint16_t*>(src) + i);
  return uint4{w.x, w.y, 0u, 0u};
}
__device__ __forceinline__ float4 Widen4(uint4 w, int dtype) {
  if (dtype == YAHKV_F32)
    return float4{__builtin_bit_cast(float, w.x), __builtin_bit_cast(float, w.y), __builtin_bit_cast(float, w.z),
                  __builtin_bit_cast(float, w.w)};
  const uint16_t h[4] = {static_cast<uint16_t>(w.x & 0xFFFF), static_cast<uint16_t>(w.x >> 16),
                         static_cast<uint16_t>(w.y & 0xFFFF), static_cast<uint16_t>(w.y >> 16)};
  if (dtype == YAHKV_F16) return float4{WidenF16(h[0]), WidenF16(h[1]), WidenF16(h[2]), WidenF16(h[3])};
  return float4{WidenBf16(h[0]), WidenBf16(h[1]), WidenBf16(h[2]), WidenBf16(h[3])};
}
// One element the same way: the raw bits (the low 16 for f16 / bf16), widened later.
__device__ __forceinline__ uint32_t LoadRaw1(const void* src, size_t i, int dtype) {
  if (dtype == YAHKV_F32) return static_cast<const uint32_t*>(src)[i];
  return static_cast<const uint16_t*>(src)[i];
}
__device__ __forceinline__ float Widen1(uint32_t w, int dtype) {
  if (dtype == YAHKV_F32) return __builtin_bit_cast(float, w);
  return dtype == YAHKV_F16 ? WidenF16(static_cast<uint16_t>(w)) : WidenBf16(static_cast<uint16_t>(w));
}

// Where a quantized row goes. A row of head_dim values lies across a wavefront, four consecutive dims per lane (lanes
// at or past head_dim / 4 hold nothing and must not call these); block b is lanes 8 b .. 8 b + 7 and `codes` is what
// the quantizers above return for the lane. K: codes [page][H][block][slot][32 | 16], scales [page][H][slot][block];
// V: codes transposed, [page][H][dim][slot] (q8_0) or [page][H][block][16][slot] (q4_0, a byte per pair of dims),
// scales [page][H][block][slot].
template <int FMT>
__device__ __forceinline__ void StoreRowK(const Pools& pools, const Geom& g, int page, int h, int slot, int lane,
                                          uint32_t codes, uint16_t scale) {
  const int NB = g.nb(), PT = g.pt, b = lane / 8, lb = lane % 8;
  const size_t ph = size_t(page) * g.n_kv + h;
  if (lb == 0) pools.ks[(ph * PT + slot) * NB + b] = scale;
  if (FMT == 8)
    *reinterpret_cast<uint32_t*>(pools.kq + ((ph * NB + b) * PT + slot) * 32 + 4 * lb) = codes;
  else if (lb < 4)
    *reinterpret_cast<uint32_t*>(pools.kq + ((ph * NB + b) * PT + slot) * 16 + 4 * lb) = codes;
}
template <int FMT>
__device__ __forceinline__ void StoreRowV(const Pools& pools, const Geom& g, int page, int h, int slot, int lane,
                                          uint32_t codes, uint16_t scale) {
  const int NB = g.nb(), PT = g.pt, b = lane / 8, lb = lane % 8;
  const size_t ph = size_t(page) * g.n_kv + h;
  if (lb == 0) pools.vs[(ph * NB + b) * PT + slot] = scale;
  if (FMT == 8) {  // row (32 b + 4 lb + e) of [D][PT]
    uint8_t* dst = pools.vq + (ph * g.hd + 4 * lane) * PT + slot;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[size_t(e) * PT] = static_cast<uint8_t>(codes >> (8 * e));
  } else if (lb < 4) {  // row (16 b + 4 lb + e) of [NB * 16][PT]
    uint8_t* dst = pools.vq + ((ph * NB + b) * 16 + 4 * lb) * PT + slot;
#pragma unroll
    for (int e = 0; e < 4; ++e) dst[size_t(e) * PT] = static_cast<uint8_t>(codes >> (8 * e));
  }
}

}  // namespace yahkv

#endif  // YAHKV_QUANT_HPP_
