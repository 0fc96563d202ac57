// The reference's own KV format, kv8a16 (docs/architecture.md:214-230), for gfx950: buffer layouts and the codec's
// arithmetic, shared by the append, decode and prefill kernels of that format.
//
//   K   int8 around a per-channel mean m, one scale per (token, kv head, 128-dim half):
//         x = f32(f16(k)) - m, s = amax / 127 (0 -> 1), u = rne(x * (1 / s)) + 128       (gen_kvq.py:166-285)
//       kq  u32 [row][H * 64]   row = page * 256 + position % 256; bytes of a dword in the order (d0, d2, d1, d3)
//       ks  u32 [row][H * 2]    f16x2 (256 s, -384 s)
//       the decode attention reads (u - 128) * (f32(f16(256 s)) / 256) in f32 (gen_decode_attn.py:784-804), the
//       prefill attention f16(1 + u / 256) * f16(256 s) + f16(-384 s) as one f16 fma (gen_attn_fa.py:4648-4773)
//   V   uint8 per channel per 16-key tile around the tile's midrange:
//         c = (max + min) / 2, s = (max - min) / 254 (0 -> 1), both rounded to f16 first (cf, sf),
//         u = clamp(rne((v - cf) * (1 / sf)) + 128, 0, 255)                              (gen_kvq.py:474-660)
//       vq  u32 [H][tile][256][4]   tile = page * 16 + (position / 16) % 16; dword w: keys 4 w + (0, 2, 1, 3)
//       vs  u32 [H][tile][256]      f16x2 (S, C') = (256 sf, cf - 384 sf)
//       decode: u * (S / 256) + (S + C') in f32 (gen_decode_attn.py:969-997); prefill: f16(1 + u / 256) * S + C'
//       The newest tile of a sequence stays open in f16 and is quantized when its 16th key arrives
//       (gen_decode_attn.py:436-573).
// The reference serves one sequence and keeps one mean vector and one open tile per decoder; here every page has a
// place for both: km f32 [page][H * 256] holds the means of the sequence whose FIRST page it is, vo f16
// [page][H * 256][16] the open tile of the sequence whose NEWEST page it is. They follow the page through forks and
// slots like the page's codes do.
#ifndef YAHKV_KV8_HPP_
#define YAHKV_KV8_HPP_

#include <type_traits>

#include "common.hpp"
#include "quant.hpp"

namespace yahkv {

constexpr int kKv8Dim = 256, kKv8Page = 256, kKv8Tile = 16;

struct Kv8Pools {
  uint32_t* kq;
  uint32_t* ks;
  float* km;
  uint32_t* vq;
  uint32_t* vs;
  uint16_t* vo;
};
inline Kv8Pools MakeKv8Pools(const yahkv_kv8_pools& p) {
  return Kv8Pools{static_cast<uint32_t*>(p.kq), static_cast<uint32_t*>(p.ks), static_cast<float*>(p.km),
                  static_cast<uint32_t*>(p.vq), static_cast<uint32_t*>(p.vs), static_cast<uint16_t*>(p.vopen)};
}

// bits of the K and of the V codes of a format of this family (0: not one of them)
__host__ __device__ inline int Kv8BitsK(int format) { return format == YAHKV_KV8A16 || format == YAHKV_K8V4A16 ? 8 : format == YAHKV_KV4A16 || format == YAHKV_K4V8A16 ? 4 : 0; }
__host__ __device__ inline int Kv8BitsV(int format) { return format == YAHKV_KV8A16 || format == YAHKV_K4V8A16 ? 8 : format == YAHKV_KV4A16 || format == YAHKV_K8V4A16 ? 4 : 0; }

int CheckKv8Geometry(const yahkv_geometry* g);
int CheckKv8Pools(const yahkv_geometry* g, const yahkv_kv8_pools* pools);

__device__ __forceinline__ uint16_t F16Bits(float x) { return __builtin_bit_cast(uint16_t, static_cast<_Float16>(x)); }
__device__ __forceinline__ float TruncF16(float x) { return static_cast<float>(static_cast<_Float16>(x)); }
// An f32 value as it is, for the conversion that follows: without this the compiler may fold a multiply and the
// conversion to f16 into one mixed-precision instruction that rounds once, where the reference rounds the product to
// f32 first and then to f16 (one f16 step apart in about one value of ten thousand).
__device__ __forceinline__ float RoundedF32(float x) {
  asm volatile("" : "+v"(x));
  return x;
}
// a rounded value as its code byte (v_cvt_i32_f32 semantics: NaN gives 0)
__device__ __forceinline__ uint32_t Kv8Byte(float r) { return static_cast<uint32_t>(static_cast<int>(r)) & 0xFFu; }

// K: the scale of a 128-dim half from its amax, as (s, 1 / s), and the half's pair (256 s, -384 s) as a dword.
__device__ __forceinline__ float Kv8ScaleK(float amax, float* inv, uint32_t* pair) {
#pragma clang fp contract(off)
  const float s0 = amax / 127.0f;
  const float s = s0 > 0.0f ? s0 : 1.0f;
  *inv = 1.0f / s;
  *pair = uint32_t(F16Bits(RoundedF32(s * 256.0f))) | (uint32_t(F16Bits(RoundedF32(s * -384.0f))) << 16);
  return s;
}
// four consecutive dims (already centred) to their dword: byte slots (d0, d2, d1, d3)
__device__ __forceinline__ uint32_t Kv8CodesK(float4 x, float inv) {
#pragma clang fp contract(off)
  const uint32_t u0 = Kv8Byte(__builtin_rintf(x.x * inv) + 128.0f), u1 = Kv8Byte(__builtin_rintf(x.y * inv) + 128.0f);
  const uint32_t u2 = Kv8Byte(__builtin_rintf(x.z * inv) + 128.0f), u3 = Kv8Byte(__builtin_rintf(x.w * inv) + 128.0f);
  return u0 | (u2 << 8) | (u1 << 16) | (u3 << 24);
}

// V: one channel's 16 keys (f32 values of f16 numbers) to its four code dwords and its stats dword.
__device__ __forceinline__ void Kv8QuantTile(const float (&x)[16], uint4* codes, uint32_t* stats) {
#pragma clang fp contract(off)
  float mx = x[0], mn = x[0];
#pragma unroll
  for (int j = 1; j < 16; ++j) mx = __builtin_fmaxf(mx, x[j]), mn = __builtin_fminf(mn, x[j]);
  const float cen = (mx + mn) * 0.5f;
  const float s0 = (mx - mn) / 254.0f;
  const float s = s0 > 0.0f ? s0 : 1.0f;
  const float sf = TruncF16(s), cf = TruncF16(cen);  // the stats are rounded to f16 before they are used
  const float inv = 1.0f / sf;
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    uint32_t u[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float r = __builtin_rintf((x[4 * i + e] - cf) * inv) + 128.0f;
      u[e] = Kv8Byte(__builtin_fminf(__builtin_fmaxf(r, 0.0f), 255.0f));  // fmaxf(NaN, 0) = 0
    }
    w[i] = u[0] | (u[2] << 8) | (u[1] << 16) | (u[3] << 24);
  }
  *codes = uint4{w[0], w[1], w[2], w[3]};
  *stats = uint32_t(F16Bits(RoundedF32(sf * 256.0f))) | (uint32_t(F16Bits(RoundedF32(cf + sf * -384.0f))) << 16);  // sf * 384 is exact
}

// ---- kv4a16 (gen_kvq.py:288-463, gen_vqt(4)) ---------------------------------------------------------------------------
//   K   H256 (k - m) / 16 per kv head, 16 levels per 32-dim group: u = clamp(rne((x - lo) * (1 / s)), 0, 15),
//       s = (hi - lo) / 15 (0 -> 1); kq u32 [row][H * 32], dims 2 j / 2 j + 1 of a dword's eight at bits 4 j / 16 + 4 j;
//       ks u32 [row][H * 8] f16x2 (S, C) = (16 s, lo - 16 s); value = (1 + u / 16) * S + C
//   V   15 levels per channel and 16-key tile: u = clamp(rne((v - cf) * (1 / sf)) + 7, 0, 14), s = range / 14;
//       vq u32 [H][tile][256][2], dword w: keys 8 w + (0, 2, 4, 6, 1, 3, 5, 7) at nibbles 0 .. 7; vs (16 sf, cf - 23 sf)

// The 256 values of a kv head across a wave, four consecutive ones per lane: H256 x, unnormalized, with the
// reference's order of f32 operations: stages 1, 2, 4 .. 128, lower' = lower + upper, upper' = lower - upper.
__device__ __forceinline__ float4 WaveHadamard256(float4 x, int lane) {
#pragma clang fp contract(off)
  const float a0 = x.x + x.y, a1 = x.x - x.y, a2 = x.z + x.w, a3 = x.z - x.w;
  float v[4] = {a0 + a2, a1 + a3, a0 - a2, a1 - a3};
  auto stage = [&](auto kc) {
    constexpr int k = decltype(kc)::value;
    const float sign = (lane & k) != 0 ? -1.0f : 1.0f;  // upper' = partner - own, lower' = own + partner
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf(v[e], sign, LaneXor<k>(v[e]));  // (+-1 * x is exact: one rounding, the sum's)
  };
  stage(std::integral_constant<int, 1>{}), stage(std::integral_constant<int, 2>{}), stage(std::integral_constant<int, 4>{});
  stage(std::integral_constant<int, 8>{}), stage(std::integral_constant<int, 16>{}), stage(std::integral_constant<int, 32>{});
  return float4{v[0], v[1], v[2], v[3]};
}

// One K row of a kv head, centred, four dims per lane: rotate, quantize per 32-dim group (eight lanes). Returns this
// lane's four codes at their places in the dword it shares with its neighbour (lanes 2 i and 2 i + 1 hold the two halves
// of dword i: `or` them), the group's pair in *pair, and what the codes decode to in f32 (u * (S / 16) + (C + S), the
// decode side's form, gen_decode_attn.py:806-850) in *deq.
__device__ __forceinline__ uint32_t Kv4CodesK(float4 centred, int lane, uint32_t* pair, float4* deq) {
#pragma clang fp contract(off)
  const float4 h = WaveHadamard256(centred, lane);
  const float xr[4] = {h.x * 0.0625f, h.y * 0.0625f, h.z * 0.0625f, h.w * 0.0625f};
  float lo = fminf(fminf(xr[0], xr[1]), fminf(xr[2], xr[3])), hi = fmaxf(fmaxf(xr[0], xr[1]), fmaxf(xr[2], xr[3]));
  lo = fminf(lo, LaneXor<1>(lo)), hi = fmaxf(hi, LaneXor<1>(hi));  // over the group's eight lanes
  lo = fminf(lo, LaneXor<2>(lo)), hi = fmaxf(hi, LaneXor<2>(hi));
  lo = fminf(lo, LaneXor<4>(lo)), hi = fmaxf(hi, LaneXor<4>(hi));
  const float s0 = (hi - lo) / 15.0f;
  const float s = s0 > 0.0f ? s0 : 1.0f;
  const float inv = 1.0f / s;
  const float S0 = RoundedF32(s * 16.0f);
  const uint32_t sb = F16Bits(S0), cb = F16Bits(RoundedF32(lo - S0));
  *pair = sb | (cb << 16);
  const float Sf = WidenF16(static_cast<uint16_t>(sb)), Cf = WidenF16(static_cast<uint16_t>(cb));
  const float d = Sf * 0.0625f, l0 = Cf + Sf;
  uint32_t w = 0;
  float dq[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const float r = __builtin_fminf(__builtin_fmaxf(__builtin_rintf((xr[e] - lo) * inv), 0.0f), 15.0f);
    const uint32_t u = static_cast<uint32_t>(static_cast<int>(r)) & 15u;
    const int i = 4 * (lane & 1) + e;  // the dim's place among the dword's eight
    w |= u << (4 * (i / 2) + (i % 2 ? 16 : 0));
    dq[e] = static_cast<float>(u) * d + l0;
  }
  *deq = float4{dq[0], dq[1], dq[2], dq[3]};
  return w;
}

// V: one channel's 16 keys to its two code dwords and its stats dword.
__device__ __forceinline__ void Kv4QuantTile(const float (&x)[16], uint2* codes, uint32_t* stats) {
#pragma clang fp contract(off)
  float mx = x[0], mn = x[0];
#pragma unroll
  for (int j = 1; j < 16; ++j) mx = __builtin_fmaxf(mx, x[j]), mn = __builtin_fminf(mn, x[j]);
  const float cen = (mx + mn) * 0.5f;
  const float s0 = (mx - mn) / 14.0f;
  const float s = s0 > 0.0f ? s0 : 1.0f;
  const float sf = TruncF16(s), cf = TruncF16(cen);
  const float inv = 1.0f / sf;
  uint32_t w[2] = {0u, 0u};
#pragma unroll
  for (int j = 0; j < 16; ++j) {
    const float r = __builtin_rintf((x[j] - cf) * inv) + 7.0f;
    const uint32_t u = static_cast<uint32_t>(static_cast<int>(__builtin_fminf(__builtin_fmaxf(r, 0.0f), 14.0f))) & 15u;
    const int k = j % 8;  // key 8 w + k: even keys at nibbles 0 .. 3, odd ones at 4 .. 7
    w[j / 8] |= u << (4 * (k % 2 ? 4 + k / 2 : k / 2));
  }
  *codes = uint2{w[0], w[1]};
  *stats = uint32_t(F16Bits(RoundedF32(sf * 16.0f))) | (uint32_t(F16Bits(RoundedF32(cf + sf * -23.0f))) << 16);  // sf * 23 is exact
}

// Layout offsets (elements of the respective arrays); kb / vb: bits of the K and of the V codes.
struct Kv8Geom {
  int32_t n_q, n_kv, n_pages, kb, vb;
  __host__ __device__ int W() const { return n_kv * kKv8Dim; }
  __host__ __device__ size_t tiles() const { return size_t(n_pages) * 16; }
  __host__ __device__ int kq_head() const { return kb == 4 ? 32 : 64; }  // dwords of a kv head's K row
  __host__ __device__ int ks_head() const { return kb == 4 ? 8 : 2; }    // scale pairs of a kv head's K row
  __host__ __device__ int vq_dim() const { return vb == 4 ? 2 : 4; }     // dwords of a (tile, dim)
  __host__ __device__ size_t kq_row(size_t row, int h) const { return (row * n_kv + h) * kq_head(); }            // dwords
  __host__ __device__ size_t ks_row(size_t row, int h) const { return (row * n_kv + h) * ks_head(); }             // dwords
  __host__ __device__ size_t vq_tile(int h, size_t pt) const { return (size_t(h) * tiles() + pt) * 256 * vq_dim(); }  // dwords
  __host__ __device__ size_t vs_tile(int h, size_t pt) const { return (size_t(h) * tiles() + pt) * 256; }   // dwords
  __host__ __device__ size_t vo_head(int page, int h) const { return (size_t(page) * n_kv + h) * 256 * 16; }  // f16
  __host__ __device__ size_t km_head(int page, int h) const { return (size_t(page) * n_kv + h) * 256; }
};
inline Kv8Geom MakeKv8Geom(const yahkv_geometry& g) {
  return Kv8Geom{g.n_q_heads, g.n_kv_heads, g.n_pages, Kv8BitsK(g.format), Kv8BitsV(g.format)};
}

}  // namespace yahkv

#endif  // YAHKV_KV8_HPP_
