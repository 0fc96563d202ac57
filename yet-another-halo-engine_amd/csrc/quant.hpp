// Block quantizers and the store of one block into its page, shared by the append kernels.
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

// A code from x * inv as the x86-64 reference computes it: lround, whose result for a non-finite or out-of-range
// argument converts to the int8 0 there (only reachable when 1 / d overflowed, i.e. amax < 2^-119).
__device__ __forceinline__ int CodeQ8(float r) { return fabsf(r) <= 128.0f ? static_cast<int>(roundf(r)) : 0; }

// 32 values -> codes (32 bytes for q8_0, 16 bytes for q4_0: element j low nibble, j + 16 high nibble) and f16 scale.
template <int FMT>
__device__ __forceinline__ void QuantizeBlock(const float (&x)[32], uint8_t (&code)[32], uint16_t* scale) {
#pragma clang fp contract(off)
  if (FMT == 8) {
    float amax = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) amax = fmaxf(amax, fabsf(x[j]));
    const float d = amax / 127.0f;
    const float inv = d > 0.0f ? 1.0f / d : 0.0f;
    *scale = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d));
#pragma unroll
    for (int j = 0; j < 32; ++j) code[j] = static_cast<uint8_t>(static_cast<int8_t>(CodeQ8(x[j] * inv)));
  } else {
    float amax = 0.0f, mx = 0.0f;
#pragma unroll
    for (int j = 0; j < 32; ++j) {
      const float av = fabsf(x[j]);
      if (amax < av) amax = av, mx = x[j];
    }
    const float d = mx / -8.0f;
    const float id = d != 0.0f ? 1.0f / d : 0.0f;
    *scale = __builtin_bit_cast(uint16_t, static_cast<_Float16>(d));
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int q0 = min(15, static_cast<int>(static_cast<int8_t>(static_cast<int>(x[j] * id + 8.5f))));
      const int q1 = min(15, static_cast<int>(static_cast<int8_t>(static_cast<int>(x[j + 16] * id + 8.5f))));
      code[j] = static_cast<uint8_t>(q0 | (q1 << 4));
    }
  }
}

// Block b of kv head h of the token in slot t of `page`: the K block is stored as 16-byte writes, the V block's
// bytes go to 32 (16) rows of the transposed page.
template <int FMT>
__device__ __forceinline__ void StoreBlock(const Geom& g, const Pools& pools, bool is_v, int page, int t, int h, int b,
                                           const uint8_t (&code)[32], uint16_t scale) {
  constexpr int CB = FMT == 8 ? 32 : 16;
  const int NB = g.nb(), H = g.n_kv, PT = g.pt;
  const size_t ph = size_t(page) * H + h;
  if (!is_v) {
    pools.ks[(ph * PT + t) * NB + b] = scale;
    uint4* dst = reinterpret_cast<uint4*>(pools.kq + ((ph * NB + b) * PT + t) * CB);
    const uint4* c4 = reinterpret_cast<const uint4*>(code);
#pragma unroll
    for (int j = 0; j < CB / 16; ++j) dst[j] = c4[j];
  } else {
    pools.vs[(ph * NB + b) * PT + t] = scale;
    // q8_0: row (32 b + j) of [D][PT]; q4_0: row (16 b + j) of [NB * 16][PT]
    uint8_t* dst = pools.vq + (ph * NB + b) * CB * PT + t;
#pragma unroll
    for (int j = 0; j < CB; ++j) dst[size_t(j) * PT] = code[j];
  }
}

}  // namespace yahkv

#endif  // YAHKV_QUANT_HPP_
