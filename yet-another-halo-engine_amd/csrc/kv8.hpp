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

#include "common.hpp"

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

// Layout offsets (elements of the respective arrays).
struct Kv8Geom {
  int32_t n_q, n_kv, n_pages;
  __host__ __device__ int W() const { return n_kv * kKv8Dim; }
  __host__ __device__ size_t tiles() const { return size_t(n_pages) * 16; }
  __host__ __device__ size_t kq_row(size_t row, int h) const { return (row * n_kv + h) * 64; }            // dwords
  __host__ __device__ size_t ks_row(size_t row, int h) const { return (row * n_kv + h) * 2; }             // dwords
  __host__ __device__ size_t vq_tile(int h, size_t pt) const { return (size_t(h) * tiles() + pt) * 1024; }  // dwords
  __host__ __device__ size_t vs_tile(int h, size_t pt) const { return (size_t(h) * tiles() + pt) * 256; }   // dwords
  __host__ __device__ size_t vo_head(int page, int h) const { return (size_t(page) * n_kv + h) * 256 * 16; }  // f16
  __host__ __device__ size_t km_head(int page, int h) const { return (size_t(page) * n_kv + h) * 256; }
};
inline Kv8Geom MakeKv8Geom(const yahkv_geometry& g) { return Kv8Geom{g.n_q_heads, g.n_kv_heads, g.n_pages}; }

}  // namespace yahkv

#endif  // YAHKV_KV8_HPP_
