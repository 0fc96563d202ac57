// Shared by the host entry points and the gfx950 kernels: geometry, the pool layout of include/yahkv.h as
// offset functions, and source-type widening.
#ifndef YAHKV_COMMON_HPP_
#define YAHKV_COMMON_HPP_

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

#include "yahkv.h"

namespace yahkv {

// Geometry as the kernels take it (by value, in SGPRs).
struct Geom {
  int32_t format, n_q, n_kv, hd, pt, n_pages;
  __host__ __device__ int nb() const { return hd / 32; }
  __host__ __device__ int group() const { return n_q / n_kv; }
  __host__ __device__ int code_bytes() const { return format == 8 ? 32 : 16; }  // per block
  // bytes of one page in the code pools / elements of one page in the scale pools
  __host__ __device__ size_t code_page() const { return size_t(n_kv) * nb() * pt * code_bytes(); }
  __host__ __device__ size_t scale_page() const { return size_t(n_kv) * pt * nb(); }
};

struct Pools {
  uint8_t* kq;
  uint16_t* ks;
  uint8_t* vq;
  uint16_t* vs;
};

inline Geom MakeGeom(const yahkv_geometry& g) {
  return Geom{g.format, g.n_q_heads, g.n_kv_heads, g.head_dim, g.page_tokens, g.n_pages};
}
inline Pools MakePools(const yahkv_pools& p) {
  return Pools{static_cast<uint8_t*>(p.kq), static_cast<uint16_t*>(p.ks), static_cast<uint8_t*>(p.vq),
               static_cast<uint16_t*>(p.vs)};
}

// Pages read from device memory are clamped into the pool (the reference's writers do: gen_kvq.py:60-71).
__device__ __forceinline__ int ClampPage(int pg, int n_pages) { return min(max(pg, 0), n_pages - 1); }

__device__ __forceinline__ float WidenBf16(uint16_t h) { return __uint_as_float(uint32_t(h) << 16); }
__device__ __forceinline__ float WidenF16(uint16_t h) {
  return static_cast<float>(__builtin_bit_cast(_Float16, h));
}
// Element i of a source array of yahkv_dtype dt, as f32 (exact).
__device__ __forceinline__ float LoadSrc(const void* p, size_t i, int dt) {
  if (dt == YAHKV_F32) return static_cast<const float*>(p)[i];
  const uint16_t h = static_cast<const uint16_t*>(p)[i];
  return dt == YAHKV_F16 ? WidenF16(h) : WidenBf16(h);
}

// Loads of pool data that a kernel reads once: the non-temporal hint. A plain streaming read of 5 GB runs at 6.0 -
// 6.2 TB/s on this chip, the same read with the hint at 6.8 - 7.0 TB/s (measured, 2048 waves with 16 KB in flight
// each). kStreamed is the hint as the cache-policy operand of the buffer and LDS-direct load builtins.
constexpr int kStreamed = 2;
template <typename T>
__device__ __forceinline__ T StreamLoad(const T* p) {  // T: 4, 8 or 16 bytes, aligned to its size
  static_assert(sizeof(T) == 4 || sizeof(T) == 8 || sizeof(T) == 16, "one, two or four dwords");
  if constexpr (sizeof(T) == 4) {
    return __builtin_bit_cast(T, __builtin_nontemporal_load(reinterpret_cast<const uint32_t*>(p)));
  } else {
    typedef uint32_t Words __attribute__((ext_vector_type(sizeof(T) / 4)));
    return __builtin_bit_cast(T, __builtin_nontemporal_load(reinterpret_cast<const Words*>(p)));
  }
}

int CheckGeometry(const yahkv_geometry* g);
// Geometry, then the four pools: not null, 16-byte aligned, each at least as long as the geometry needs.
int CheckPools(const yahkv_geometry* g, const yahkv_pools* pools);
inline int LaunchStatus() { return hipGetLastError() == hipSuccess ? YAHKV_OK : YAHKV_ERR_LAUNCH; }

}  // namespace yahkv

#endif  // YAHKV_COMMON_HPP_
