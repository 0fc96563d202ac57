// Chunked-prefill attention over the paged, block-quantized prefix: a FlashAttention-style kernel on 16-bit MFMA.
//
// Semantics follow the reference's prefill attention (engine/gpu/loom/tools/gen_attn_fa.py:1-21, launch signature
// :1589-1595): query t of the chunk sees keys 0 .. prefix + t, which the caller has already appended to the pools;
// online softmax in base 2 (:1614), output o / l, times sigmoid(gate) if a gate is given (:4230). Quantized K / V are
// decoded while they are staged into LDS (:2664-2779) to f16, as the reference's kernel computes in f16 (:1252-1595):
// value = f16(d * code), round to nearest even, saturated at the largest finite f16 (d * code can reach 65504 * 127).
// The chunk's bf16 queries become f16 the same way (exact in the normal f16 range), and so do the softmax numerators.
// f16 and bf16 run at the same MFMA rate; f16's three more mantissa bits are what brings the result within 2e-3 of
// exact arithmetic on 18K keys (bf16 keys alone cost 1.5e-3 there).
//
// Shape of the computation (everything is transposed so that keys run along MFMA rows and queries along lanes):
//   S^T[key][q] = sum_dim K[key][dim] Q[q][dim]     A = K tile from LDS (16 keys x 32 dims), B = Q^T (registers)
//   O^T[dim][q] += sum_key V^T[dim][key] P^T[key][q]  A = V^T tile from LDS (16 dims x 32 keys), B = P^T (registers)
// v_mfma_f32_16x16x32_f16 leaves S^T with one query per lane and keys down the registers, which is exactly the
// B-operand shape of the second product: P never leaves the registers, the row maximum needs two cross-lane steps, and
// the rescaling factor of a lane's accumulators is the lane's own.
// A workgroup (4 waves) owns 64 consecutive chunk positions of one sequence for two query heads of one kv head: eight
// row blocks of 16 queries, two per wave (three per wave would let all six heads of a group share a tile, but the
// accumulators of three blocks at head_dim 256, 192 registers, leave too little room and the kernel spills). Every
// K / V tile is fetched and decoded once per workgroup and used by all eight blocks (the reference decodes once per
// layer into an f16 pool for the same reason, :4648-4861).
#include "common.hpp"
#include "kv8.hpp"

namespace yahkv {
namespace {

constexpr int kKeys = 64;    // keys per tile
constexpr int kQueries = 64; // chunk positions per workgroup
constexpr int kFusedRowBlocks = 2;  // row blocks (16 queries of one head) per wave of the one-pass kernel
constexpr float kNegBig = -3.4028234663852886e+38f;

typedef _Float16 h8v __attribute__((ext_vector_type(8)));
// The softmax numerators are 2^(score - m) with a reference point m that sits kBias below the (rounded-up) largest
// score seen when it was set and is moved when a score exceeds it by more than kBias + kSlack: the numerators then
// stay below 2^(kBias + kSlack), well inside f16's range, while a numerator 2^-24 of the largest is still a normal
// f16. Numerators and denominators carry the same factor, so it cancels.
constexpr float kBias = 10.0f, kSlack = 4.0f;
typedef float f4v __attribute__((ext_vector_type(4)));

struct PrefillArgs {
  Geom g;
  Pools pools;
  const int32_t* table;
  int32_t stride;
  const int32_t* prefix_len;
  int32_t n_seqs, max_prefix, chunk_len;
  const uint16_t* q;  // bf16 [n_seqs][chunk_len][n_q][D]
  int32_t q_is_f16;   // q holds f16 values instead (the rotated queries of the 4-bit K format)
  float scale;
  const float* gate;
  void* out;
  int32_t out_dtype;
};

__device__ __forceinline__ h8v OnesF16() {  // 1.0 in all eight slots
  return __builtin_bit_cast(h8v, uint4{0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u});
}
typedef _Float16 h2v __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t PackF16(float a, float b) {  // round to nearest even (one v_cvt_pk_f16_f32)
  const h2v v = {static_cast<_Float16>(a), static_cast<_Float16>(b)};
  return __builtin_bit_cast(uint32_t, v);
}
// For K and V values: finite values beyond the f16 range saturate at +-65504 (NaN stays NaN).
__device__ __forceinline__ float ClampF16(float x) { return __builtin_fminf(__builtin_fmaxf(x, -65504.0f), 65504.0f) + (x - x); }
__device__ __forceinline__ uint32_t PackF16Sat(float a, float b) { return PackF16(ClampF16(a), ClampF16(b)); }
// Eight bf16 query elements as f16.
__device__ __forceinline__ h8v QueryF16(const uint16_t* p, bool is_f16 = false) {
  const uint4 w = *reinterpret_cast<const uint4*>(p);
  if (is_f16) return __builtin_bit_cast(h8v, w);
  const uint32_t u[4] = {w.x, w.y, w.z, w.w};
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = PackF16Sat(WidenBf16(static_cast<uint16_t>(u[e] & 0xFFFF)), WidenBf16(static_cast<uint16_t>(u[e] >> 16)));
  return __builtin_bit_cast(h8v, uint4{o[0], o[1], o[2], o[3]});
}
__device__ __forceinline__ uint32_t PackBf16(float a, float b) {  // round to nearest even
  typedef __bf16 b2v __attribute__((ext_vector_type(2)));
  const b2v v = {static_cast<__bf16>(a), static_cast<__bf16>(b)};
  return __builtin_bit_cast(uint32_t, v);
}

// Sixteen codes times one scale, as sixteen f16 (two 16-byte halves). q8_0: sixteen int8 codes. q4_0: the low
// (SHIFT 0) or high (SHIFT 4) nibbles of a block's sixteen bytes, value (n - 8) * d.
template <int FMT>
__device__ __forceinline__ void Decode16(const uint4 c, float d, int shift, uint4* lo, uint4* hi) {
  uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = FMT == 8 ? w[i] ^ 0x80808080u : (w[i] >> shift) & 0x0F0F0F0Fu;
  const float off = (FMT == 8 ? -128.0f : -8.0f) * d;
  uint32_t o[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {  // v_cvt_f32_ubyteN on code + 128, then one fma brings it back and scales it
    const float f0 = __builtin_fmaf(static_cast<float>(w[i] & 0xFF), d, off);
    const float f1 = __builtin_fmaf(static_cast<float>((w[i] >> 8) & 0xFF), d, off);
    const float f2 = __builtin_fmaf(static_cast<float>((w[i] >> 16) & 0xFF), d, off);
    const float f3 = __builtin_fmaf(static_cast<float>(w[i] >> 24), d, off);
    o[2 * i] = PackF16Sat(f0, f1), o[2 * i + 1] = PackF16Sat(f2, f3);
  }
  *lo = uint4{o[0], o[1], o[2], o[3]}, *hi = uint4{o[4], o[5], o[6], o[7]};
}
// Sixteen codes of one dim, sixteen keys, each with its own scale (q4_0: one nibble of the sixteen bytes of a byte row).
template <int FMT>
__device__ __forceinline__ void Decode16V(const uint4 c, const uint4 s0, const uint4 s1, int shift, uint4* lo, uint4* hi) {
  uint32_t w[4] = {c.x, c.y, c.z, c.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = FMT == 8 ? w[i] ^ 0x80808080u : (w[i] >> shift) & 0x0F0F0F0Fu;
  constexpr float kZero = FMT == 8 ? -128.0f : -8.0f;
  const uint32_t sw[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
  uint32_t o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float d0 = WidenF16(static_cast<uint16_t>(sw[i] & 0xFFFF)), d1 = WidenF16(static_cast<uint16_t>(sw[i] >> 16));
    const uint32_t b0 = (w[i / 2] >> (16 * (i % 2))) & 0xFF, b1 = (w[i / 2] >> (16 * (i % 2) + 8)) & 0xFF;
    o[i] = PackF16Sat(__builtin_fmaf(static_cast<float>(b0), d0, kZero * d0),
                      __builtin_fmaf(static_cast<float>(b1), d1, kZero * d1));
  }
  *lo = uint4{o[0], o[1], o[2], o[3]}, *hi = uint4{o[4], o[5], o[6], o[7]};
}

// out = o / l (* sigmoid(gate)); lane (query, lane group jg) holds dims 16 dt + 4 jg + r of its query in each row block.
// The denominators l are the sums of the f16 numerators, accumulated by the matrix unit against an all-ones operand
// next to V^T: numerators and denominator then carry the same rounding, and a lone key returns its V row exactly.
// (NDT of the head's 16-dim tiles, starting with dim `dim0`: a wave that holds only part of its rows' dims)
template <int D, int RB, int NDT = D / 16>
__device__ __forceinline__ void StoreRows(const PrefillArgs& a, int s, int h, int G, int jg, const f4v (&o)[RB][NDT],
                                          const f4v (&lacc)[RB], const int (&qpos)[RB], const int (&head)[RB],
                                          int dim0 = 0) {
  const Geom& g = a.g;
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    if (head[i] >= G || qpos[i] >= a.chunk_len) continue;
    const float inv = 1.0f / lacc[i][0];  // every row of the all-ones product holds the query's denominator
    const size_t base = ((size_t(s) * a.chunk_len + qpos[i]) * g.n_q + size_t(h) * G + head[i]) * D + dim0;
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      float v[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        v[r] = o[i][dt][r] * inv;
        if (a.gate != nullptr) v[r] *= 1.0f / (1.0f + __expf(-a.gate[base + 16 * dt + 4 * jg + r]));
      }
      const size_t e = base + 16 * dt + 4 * jg;
      if (a.out_dtype == YAHKV_F32) {
        *reinterpret_cast<float4*>(static_cast<float*>(a.out) + e) = float4{v[0], v[1], v[2], v[3]};
      } else if (a.out_dtype == YAHKV_BF16) {
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.out) + e) = uint2{PackBf16(v[0], v[1]), PackBf16(v[2], v[3])};
      } else {
        typedef _Float16 h2v __attribute__((ext_vector_type(2)));
        const h2v x = {static_cast<_Float16>(v[0]), static_cast<_Float16>(v[1])};
        const h2v y = {static_cast<_Float16>(v[2]), static_cast<_Float16>(v[3])};
        *reinterpret_cast<uint2*>(static_cast<uint16_t*>(a.out) + e) =
            uint2{__builtin_bit_cast(uint32_t, x), __builtin_bit_cast(uint32_t, y)};
      }
    }
  }
}

template <int FMT, int D, int PT>
__global__ __launch_bounds__(256) void PrefillAttendFused(const PrefillArgs a) {
  constexpr int NB = D / 32, NDT = D / 16, KS = D / 32;  // blocks, 16-dim tiles, 32-dim steps of the first product
  constexpr int RB = kFusedRowBlocks, kHeadsPerGroup = RB;  // 4 waves x RB row blocks = 64 positions x RB heads
  constexpr int KSTR = D + 8, VSTR = kKeys + 8;          // LDS row strides (f16), padded against bank conflicts
  constexpr int KCH = kKeys * D / 16 / 256;              // 16-code chunks of a tile per thread
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const int n_qt = (a.chunk_len + kQueries - 1) / kQueries, n_hp = (G + kHeadsPerGroup - 1) / kHeadsPerGroup;
  // Workgroups of one (sequence, kv head) pair run on one XCD (they stream the same K / V through that XCD's L2),
  // longest query tile first.
  const int bid = blockIdx.x, xcd = bid % 8, local = bid / 8, per_pair = n_qt * n_hp;
  const int pair = xcd + 8 * (local / per_pair), qt = n_qt - 1 - (local % per_pair) / n_hp, hp = local % n_hp;
  if (pair >= a.n_seqs * H) return;
  const int s = pair / H, h = pair % H;
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int qn = lane % 16, jg = lane / 16;  // lane = query (mod 16); lane group = rows 4 jg .. 4 jg + 3 of a tile
  const int prefix = min(max(a.prefix_len[s], 0), min(a.max_prefix, a.stride * g.pt - a.chunk_len));
  const int q0 = qt * kQueries;              // first chunk position of this workgroup
  const int n_keys = min(prefix + q0 + kQueries, prefix + a.chunk_len);
  const int n_tiles = (n_keys + kKeys - 1) / kKeys;

  __shared__ __align__(16) _Float16 lk[kKeys][KSTR];  // K tile, [key][dim]
  __shared__ __align__(16) _Float16 lv[D][VSTR];      // V^T tile, [dim][key]
  __shared__ __align__(16) uint16_t lvs[NB][kKeys]; // V scales of the tile (f16 bits), [block][key]

  // ---- this wave's row blocks: rb = RB * wave + i -> head 2 hp + rb / 4, queries q0 + 16 (rb % 4) + 0..15
  h8v qb[RB][KS];
  int qpos[RB];   // chunk position of this lane's query in block i (may be >= chunk_len: then it is never stored)
  int head[RB];   // head within the group (may be >= G: then the block is never stored)
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int rb = RB * wave + i;
    head[i] = kHeadsPerGroup * hp + rb / 4;
    qpos[i] = q0 + 16 * (rb % 4) + qn;
    const int t = min(qpos[i], a.chunk_len - 1), hd = min(head[i], G - 1);
    const uint16_t* qp = a.q + ((size_t(s) * a.chunk_len + t) * g.n_q + size_t(h) * G + hd) * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qb[i][ks] = QueryF16(qp + 32 * ks + 8 * jg);
  }
  f4v o[RB][NDT];
  float m[RB];
  f4v lacc[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    m[i] = kNegBig, lacc[i] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[i][dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
  }
  const float sscale = a.scale * 1.4426950408889634f;
  const int32_t* row = a.table + int64_t(s) * a.stride;
  auto page_head = [&](int key) -> size_t {  // (page, kv head) index of a key of the sequence
    return size_t(ClampPage(row[min(key / PT, a.stride - 1)], g.n_pages)) * H + h;
  };

  // staging registers: this thread's chunks of the K tile and of the V tile that come next (fetched one tile ahead)
  uint4 kraw[KCH], vraw[KCH];
  uint16_t ksr[KCH];
  uint4 vsr;  // threads 0 .. NB * 8 - 1: eight V scales of one block
  auto fetch_k = [&](int tile) {  // chunk c: block c / 128, key (c % 128) / 2, half c % 2
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      const int c = tid + 256 * j, b = c / 128, key = (c % 128) / 2, hf = c % 2;
      const int kk = min(tile * kKeys + key, a.stride * PT - 1);
      const size_t ph = page_head(kk);
      // q8_0: this half's sixteen codes; q4_0: the block's sixteen bytes (this half is one nibble of each)
      kraw[j] = FMT == 8 ? *reinterpret_cast<const uint4*>(a.pools.kq + ((ph * NB + b) * PT + kk % PT) * 32 + 16 * hf)
                         : *reinterpret_cast<const uint4*>(a.pools.kq + ((ph * NB + b) * PT + kk % PT) * 16);
      ksr[j] = a.pools.ks[(ph * PT + kk % PT) * NB + b];
    }
  };
  auto stage_k = [&](int j) {
    const int c = tid + 256 * j, b = c / 128, key = (c % 128) / 2, hf = c % 2;
    uint4 lo, hi;
    Decode16<FMT>(kraw[j], WidenF16(ksr[j]), 4 * hf, &lo, &hi);
    uint4* dst = reinterpret_cast<uint4*>(&lk[key][32 * b + 16 * hf]);
    dst[0] = lo, dst[1] = hi;
  };
  auto fetch_v = [&](int tile) {  // chunk c: dim c / 4, keys 16 (c % 4) .. + 15
#pragma unroll
    for (int j = 0; j < KCH; ++j) {
      const int c = tid + 256 * j, d = c / 4, k0 = 16 * (c % 4);
      const int kk = min(tile * kKeys + k0, a.stride * PT - 16);
      // q4_0: byte row d % 16 of block d / 32 holds dims d % 16 (low nibbles) and 16 + d % 16 (high) of the block
      vraw[j] = FMT == 8 ? *reinterpret_cast<const uint4*>(a.pools.vq + (page_head(kk) * D + d) * PT + kk % PT)
                         : *reinterpret_cast<const uint4*>(a.pools.vq + ((page_head(kk) * NB + d / 32) * 16 + d % 16) * PT +
                                                           kk % PT);
    }
  };
  auto fetch_vs = [&](int tile) {  // the tile's V scales: thread = (block, 8 keys)
    if (tid < NB * 8) {
      const int b = tid / 8, kk = min(tile * kKeys + 8 * (tid % 8), a.stride * PT - 8);
      vsr = *reinterpret_cast<const uint4*>(a.pools.vs + (page_head(kk) * NB + b) * PT + kk % PT);
    }
  };
  // V scales to LDS; keys past the end get scale 0, so stale bytes decode to 0 and 0 * P stays 0
  auto stage_vs = [&](int tile) {
    if (tid < NB * 8) {
      uint32_t sw[4] = {vsr.x, vsr.y, vsr.z, vsr.w};
      const int kbase = tile * kKeys + 8 * (tid % 8);
      if (kbase + 8 > n_keys) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (kbase + e >= n_keys) sw[e / 2] &= e % 2 ? 0x0000FFFFu : 0xFFFF0000u;
      }
      *reinterpret_cast<uint4*>(&lvs[tid / 8][8 * (tid % 8)]) = uint4{sw[0], sw[1], sw[2], sw[3]};
    }
  };
  auto stage_v = [&](int j) {
    const int c = tid + 256 * j, d = c / 4, k0 = 16 * (c % 4);
    const uint4* sp = reinterpret_cast<const uint4*>(&lvs[d / 32][k0]);
    uint4 lo, hi;
    Decode16V<FMT>(vraw[j], sp[0], sp[1], d % 32 / 16 * 4, &lo, &hi);
    uint4* dst = reinterpret_cast<uint4*>(&lv[d][k0]);
    dst[0] = lo, dst[1] = hi;
  };

  // Pipeline: while the matrix cores run tile i's K Q^T out of lk, the vector units decode V(i) into lv; while they
  // run V^T P^T out of lv, K(i + 1) is decoded into lk. Raw bytes are fetched a whole tile before they are decoded.
  fetch_k(0);
  fetch_vs(0);
  fetch_v(0);
#pragma unroll
  for (int j = 0; j < KCH; ++j) stage_k(j);
  stage_vs(0);
  if (n_tiles > 1) fetch_k(1), fetch_vs(1);
  __syncthreads();
  for (int tile = 0; tile < n_tiles; ++tile) {
    // ---- S^T = K Q^T, keys 16 kt + 4 jg + r down the registers
    f4v st[RB][4];
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) st[i][kt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    {
      // A operands are read one 32-dim step ahead of the products that use them; the scheduling groups spread the
      // vector work of the V decode between the matrix instructions (one wave per SIMD: nothing else hides latency).
      h8v ka[2][4];
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) ka[0][kt] = *reinterpret_cast<const h8v*>(&lk[16 * kt + qn][8 * jg]);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        if (ks + 1 < KS) {
#pragma unroll
          for (int kt = 0; kt < 4; ++kt)
            ka[(ks + 1) % 2][kt] = *reinterpret_cast<const h8v*>(&lk[16 * kt + qn][32 * (ks + 1) + 8 * jg]);
        }
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int i = 0; i < RB; ++i)
            st[i][kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[ks % 2][kt], qb[i][ks], st[i][kt], 0, 0, 0);
        if (ks % (KS / KCH) == KS / KCH - 1) {
          stage_v(ks / (KS / KCH));
#pragma unroll
          for (int n = 0; n < 8; ++n) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);  // two matrix instructions
            __builtin_amdgcn_sched_group_barrier(0x002, 10, 0); // ten vector instructions
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (tile + 1 < n_tiles) fetch_v(tile + 1);
    // ---- online softmax per query (= per lane); the row maximum crosses the four lane groups
    const bool diag = (tile + 1) * kKeys > prefix + q0 + 1;  // some key of the tile is masked for some query
    uint32_t pb[RB][2][4];                                   // P^T B-operands: [32-key step][packed pairs]
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      float mx = kNegBig;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float v = st[i][kt][r] * sscale;
          if (diag && tile * kKeys + 16 * kt + 4 * jg + r > prefix + qpos[i]) v = kNegBig;
          st[i][kt][r] = v;
          mx = fmaxf(mx, v);
        }
      mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
      mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
      // The running maximum moves in whole powers of two: rescaling is then exact, so the result does not depend on
      // the order in which the maximum was met (and it moves less often).
      const float mn = fmaxf(m[i], __builtin_ceilf(mx) - kBias);
      const float alpha = __builtin_amdgcn_exp2f(m[i] - mn);
      m[i] = mn;
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) {
        float p[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(st[i][kt][r] - mn);
        // step kt / 2 takes keys 32 (kt / 2) + {4 jg + r} from its even tile and + 16 + {4 jg + r} from its odd one
        pb[i][kt / 2][2 * (kt % 2)] = PackF16(p[0], p[1]);
        pb[i][kt / 2][2 * (kt % 2) + 1] = PackF16(p[2], p[3]);
      }
      if (alpha != 1.0f) {
#pragma unroll
        for (int r = 0; r < 4; ++r) lacc[i][r] *= alpha;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[i][dt][r] *= alpha;
      }
    }
    __syncthreads();  // every wave is done with lk, and V(tile) is complete in lv
    // ---- O^T += V^T P^T; the A operand's key slots follow pb: 4 keys at 32 s2 + 4 jg, 4 at 32 s2 + 16 + 4 jg
    {
      auto read_v = [&](int dt, int s2) -> h8v {
        const uint2 v0 = *reinterpret_cast<const uint2*>(&lv[16 * dt + qn][32 * s2 + 4 * jg]);
        const uint2 v1 = *reinterpret_cast<const uint2*>(&lv[16 * dt + qn][32 * s2 + 16 + 4 * jg]);
        return __builtin_bit_cast(h8v, uint4{v0.x, v0.y, v1.x, v1.y});
      };
      h8v pv[RB][2];
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
          pv[i][s2] = __builtin_bit_cast(h8v, uint4{pb[i][s2][0], pb[i][s2][1], pb[i][s2][2], pb[i][s2][3]});
      h8v va[3][2];  // read two 16-dim tiles ahead
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) va[0][s2] = read_v(0, s2), va[1][s2] = read_v(1, s2);
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int i = 0; i < RB; ++i)
          lacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(OnesF16(), pv[i][s2], lacc[i], 0, 0, 0);
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        if (dt + 2 < NDT) {
#pragma unroll
          for (int s2 = 0; s2 < 2; ++s2) va[(dt + 2) % 3][s2] = read_v(dt + 2, s2);
        }
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
          for (int i = 0; i < RB; ++i)
            o[i][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[dt % 3][s2], pv[i][s2], o[i][dt], 0, 0, 0);
        if (dt % (NDT / KCH) == NDT / KCH - 1) {
          stage_k(dt / (NDT / KCH));  // K(tile + 1), or stale bytes after the last tile
#pragma unroll
          for (int n = 0; n < 8; ++n) {
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
            __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);
          }
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    stage_vs(tile + 1);
    if (tile + 2 < n_tiles) fetch_k(tile + 2), fetch_vs(tile + 2);
    __syncthreads();  // every wave is done with lv; K(tile + 1) and its V scales are in place
  }

  StoreRows<D, RB>(a, s, h, G, jg, o, lacc, qpos, head);
}


// ---- two passes: tile images, then attention on the images ---------------------------------------------------------------
//
// The fused kernel above decodes every K / V tile once per workgroup, i.e. once per 64 chunk positions and pair of
// heads: at 2048 positions and 6 heads per kv head that is 96 times per key, and with one wave per SIMD the decode's
// vector instructions and the matrix instructions compete for the wave's issue slots. When the caller provides a
// workspace, the prefix is decoded once per call instead (the reference does the same: yah_kdeq8 / yah_vdeq8 into an
// f16 pool before yah_attn_wmma, gen_attn_fa.py:4648-4861): `PrefillImages` writes, per (sequence, kv head, tile of
// 64 keys), the f16 K tile and V^T tile exactly as the attention kernel wants them in LDS, and `PrefillAttendImg`
// copies images to LDS with direct global-to-LDS loads (no registers, no vector instructions) one tile ahead.
//
// K image: 64 rows (keys) of D f16; the 16-byte chunk c of row r sits at chunk position c ^ (r % 16).
// V image: D rows (dims) of 64 f16; chunk c = 4 s2 + jg of row r holds keys 32 s2 + 4 jg + 0..3 and 32 s2 + 16 +
// 4 jg + 0..3 (the eight k-slots of lane group jg in step s2 of the second product) and sits at position c ^ (r % 8).
// With the XOR, the sixteen rows a wave reads at once (four 16-byte chunks of each) fall into different banks: a K
// row is a multiple of 256 bytes, the width of the LDS banks, so sixteen rows need sixteen different chunk positions
// (with c ^ (r % 8), rows r and r + 8 met in the same banks and a wave-wide read took twice as long: 33 against 17
// cycles, measured with the reads alone); V^T rows are 128 bytes, where eight positions and the rows' own alternation
// between the two halves of the banks do. Keys at or past the end of the sequence are zero in both images.
struct ImageArgs {
  Geom g;
  Pools pools;
  const int32_t* table;
  int32_t stride;
  const int32_t* prefix_len;
  int32_t n_seqs, max_prefix, chunk_len;
  char* img;
  int32_t tiles_per_pair;
  const uint16_t* fk;  // unquantized f16 pools (PrefillImagesF16 only): K [page][H][D / 16][PT][16], V^T [page][H][PT / R][D][R], R = min(PT, 32)
  const uint16_t* fv;
  Kv8Pools kv8;        // kv8a16 pools (PrefillImagesKv8 only)
};

template <int D>
constexpr int TileImageBytes() { return 2 * kKeys * D * 2; }

__device__ __forceinline__ int ClampPrefix(const int32_t* prefix_len, int s, int max_prefix, int stride, int pt,
                                           int chunk_len) {
  return min(max(prefix_len[s], 0), min(max_prefix, stride * pt - chunk_len));
}

template <int FMT, int D, int PT>
__global__ __launch_bounds__(256) void PrefillImages(const ImageArgs a) {
  constexpr int NB = D / 32, CPR = D / 8;  // blocks; 16-byte chunks per K row
  constexpr bool Q8 = FMT == 8;
  const Geom g = a.g;
  const int H = g.n_kv, tile = blockIdx.x, pair = blockIdx.y, s = pair / H, h = pair % H, tid = threadIdx.x;
  const int n_keys = ClampPrefix(a.prefix_len, s, a.max_prefix, a.stride, g.pt, a.chunk_len) + a.chunk_len;
  if (tile * kKeys >= n_keys) return;
  const int32_t* row = a.table + int64_t(s) * a.stride;
  char* kimg = a.img + (size_t(pair) * a.tiles_per_pair + tile) * TileImageBytes<D>();
  char* vimg = kimg + kKeys * D * 2;
  auto page_head = [&](int key) -> size_t {
    return size_t(ClampPage(row[min(key / PT, a.stride - 1)], g.n_pages)) * H + h;
  };
  for (int p = tid; p < kKeys * CPR; p += 256) {  // K: chunk = dims 8 c .. 8 c + 7 of one key
    const int key = p / CPR, c = (p % CPR) ^ (key % 16), kk = tile * kKeys + key;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
    if (kk < n_keys) {
      const size_t ph = page_head(kk);
      const int t = kk % PT, b = c / 4, off = (8 * c) % 32;
      const float d = WidenF16(a.pools.ks[(ph * PT + t) * NB + b]);
      float v[8];
      if constexpr (Q8) {
        const uint2 w = StreamLoad(reinterpret_cast<const uint2*>(a.pools.kq + ((ph * NB + b) * PT + t) * 32 + off));
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[e] = d * static_cast<float>(static_cast<int8_t>(((e < 4 ? w.x : w.y) >> (8 * (e % 4))) & 0xFF));
      } else {  // byte j of a block: low nibble dim j, high nibble dim 16 + j
        const uint2 w = StreamLoad(reinterpret_cast<const uint2*>(a.pools.kq + ((ph * NB + b) * PT + t) * 16 + off % 16));
#pragma unroll
        for (int e = 0; e < 8; ++e)
          v[e] = d * static_cast<float>(int((((e < 4 ? w.x : w.y) >> (8 * (e % 4))) >> (off / 16 * 4)) & 0xF) - 8);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = PackF16Sat(v[2 * e], v[2 * e + 1]);
    }
    *reinterpret_cast<uint4*>(kimg + size_t(p) * 16) = uint4{o[0], o[1], o[2], o[3]};
  }
  for (int p = tid; p < D * 8; p += 256) {  // V: chunk = 4 + 4 keys of one dim
    const int dim = p / 8, c = (p % 8) ^ (dim % 8), s2 = c / 4, jg = c % 4, b = dim / 32;
    uint32_t o[4];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      // four keys, always within one page
      const int kk = tile * kKeys + 32 * s2 + 16 * hf + 4 * jg;
      const size_t ph = page_head(kk);
      const int t = kk % PT;
      const uint2 sw = *reinterpret_cast<const uint2*>(a.pools.vs + (ph * NB + b) * PT + t);
      uint32_t w;
      int shift = 0;
      if constexpr (Q8) {
        w = StreamLoad(reinterpret_cast<const uint32_t*>(a.pools.vq + (ph * D + dim) * PT + t));
      } else {  // byte row j of a block: low nibble dim j, high nibble dim 16 + j
        w = StreamLoad(reinterpret_cast<const uint32_t*>(a.pools.vq + ((ph * NB + b) * 16 + dim % 16) * PT + t));
        shift = dim % 32 / 16 * 4;
      }
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float d = WidenF16(static_cast<uint16_t>((e < 2 ? sw.x : sw.y) >> (16 * (e % 2))));
        const uint32_t byte = (w >> (8 * e)) & 0xFF;
        const float code = Q8 ? static_cast<float>(static_cast<int8_t>(byte))
                              : static_cast<float>(int((byte >> shift) & 0xF) - 8);
        v[e] = kk + e < n_keys ? d * code : 0.0f;
      }
      o[2 * hf] = PackF16Sat(v[0], v[1]), o[2 * hf + 1] = PackF16Sat(v[2], v[3]);
    }
    *reinterpret_cast<uint4*>(vimg + size_t(p) * 16) = uint4{o[0], o[1], o[2], o[3]};
  }
}

// The same images from unquantized f16 pools (the pools of yahkv_f16_append): the pools' own f16 values, moved into
// the images' order.
template <int D, int PT>
__global__ __launch_bounds__(256) void PrefillImagesF16(const ImageArgs a) {
  constexpr int CPR = D / 8;  // 16-byte chunks per K row
  const Geom g = a.g;
  const int H = g.n_kv, tile = blockIdx.x, pair = blockIdx.y, s = pair / H, h = pair % H, tid = threadIdx.x;
  const int n_keys = ClampPrefix(a.prefix_len, s, a.max_prefix, a.stride, g.pt, a.chunk_len) + a.chunk_len;
  if (tile * kKeys >= n_keys) return;
  const int32_t* row = a.table + int64_t(s) * a.stride;
  char* kimg = a.img + (size_t(pair) * a.tiles_per_pair + tile) * TileImageBytes<D>();
  char* vimg = kimg + kKeys * D * 2;
  auto page_head = [&](int key) -> size_t {
    return size_t(ClampPage(row[min(key / PT, a.stride - 1)], g.n_pages)) * H + h;
  };
  for (int p = tid; p < kKeys * CPR; p += 256) {  // K: chunk = dims 8 c .. 8 c + 7 of one key
    const int key = p / CPR, c = (p % CPR) ^ (key % 16), kk = tile * kKeys + key;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
    if (kk < n_keys) {
      const uint4 w = StreamLoad(reinterpret_cast<const uint4*>(a.fk + page_head(kk) * (size_t(D) * PT) +
                                                                (size_t(c / 2) * PT + kk % PT) * 16 + (c % 2) * 8));
      o[0] = w.x, o[1] = w.y, o[2] = w.z, o[3] = w.w;
    }
    *reinterpret_cast<uint4*>(kimg + size_t(p) * 16) = uint4{o[0], o[1], o[2], o[3]};
  }
  for (int p = tid; p < D * 8; p += 256) {  // V: chunk = 4 + 4 keys of one dim
    const int dim = p / 8, c = (p % 8) ^ (dim % 8), s2 = c / 4, jg = c % 4;
    uint32_t o[4];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      // four keys, always within one page
      const int kk = tile * kKeys + 32 * s2 + 16 * hf + 4 * jg;
      constexpr int RUN = PT < 32 ? PT : 32;  // V^T lies in runs of at most 32 keys
      const uint2 w = StreamLoad(reinterpret_cast<const uint2*>(a.fv + page_head(kk) * (size_t(D) * PT) +
                                                                (size_t(kk % PT / RUN) * D + dim) * RUN + kk % RUN));
      uint32_t u[2] = {w.x, w.y};
#pragma unroll
      for (int e = 0; e < 4; ++e)  // keys at or past the end are zero in the image
        if (kk + e >= n_keys) u[e / 2] &= e % 2 ? 0x0000FFFFu : 0xFFFF0000u;
      o[2 * hf] = u[0], o[2 * hf + 1] = u[1];
    }
    *reinterpret_cast<uint4*>(vimg + size_t(p) * 16) = uint4{o[0], o[1], o[2], o[3]};
  }
}

// The same images from kv8a16 pools (kv8.hpp), decoded as the reference's prefill does it (yah_kdeq8 / yah_vdeq8,
// gen_attn_fa.py:4648-4861): a code u becomes the f16 1 + u / 256 by a shift and a mask (the byte order (d0, d2, d1, d3)
// makes the two masks of a dword give the pairs in order), and one f16 fma with the pair (S, C') gives the value:
// K - mean from (256 s, -384 s) of the row's 128-dim half, V from the (tile, dim) stats; every V tile from its codes.
__device__ __forceinline__ void Kv8DecodeDword(uint32_t w, uint32_t pair, uint32_t* lo, uint32_t* hi) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 sp = __builtin_bit_cast(h2, pair);
  const h2 S = {sp[0], sp[0]}, C = {sp[1], sp[1]};
  const h2 a = __builtin_bit_cast(h2, ((w << 2) & 0x03fc03fcu) | 0x3c003c00u);  // elements 0, 1 of the dword's four
  const h2 b = __builtin_bit_cast(h2, ((w >> 6) & 0x03fc03fcu) | 0x3c003c00u);  // elements 2, 3
  *lo = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(a, S, C));
  *hi = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(b, S, C));
}
// 4-bit codes (kv4a16): eight nibbles of a dword (elements 2 j / 2 j + 1 at bits 4 j / 16 + 4 j) become the f16 pairs
// 1 + u / 16 in order by four shifts and masks, and the same fma gives the values (yah_kdeq4 / yah_vdeq4,
// gen_attn_fa.py:4652-4700). `first`: the pair index of the first of the `n` pairs wanted.
__device__ __forceinline__ void Kv4DecodePairs(uint32_t w, uint32_t pair, int first, int n, uint32_t* out) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 sp = __builtin_bit_cast(h2, pair);
  const h2 S = {sp[0], sp[0]}, C = {sp[1], sp[1]};
  for (int i = 0; i < n; ++i) {
    const int sh = 6 - 4 * (first + i);  // pair 0: << 6, 1: << 2, 2: >> 2, 3: >> 6
    const uint32_t x = sh >= 0 ? w << sh : w >> -sh;
    const h2 f = __builtin_bit_cast(h2, (x & 0x03c003c0u) | 0x3c003c00u);
    out[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(f, S, C));
  }
}
// The queries of a chunk rotated for 4-bit K: f16(H256 q / 16) per head (yah_qrot, gen_attn_fa.py:4541-4611; the
// softmax scale stays a separate factor here). One wave per (token, head) row, four dims per lane.
__global__ __launch_bounds__(256) void Kv4RotateQ(const uint16_t* q, uint16_t* out, int64_t n_rows) {
#pragma clang fp contract(off)
  const int64_t r = int64_t(blockIdx.x) * 4 + threadIdx.x / 64;
  const int lane = threadIdx.x % 64;
  if (r >= n_rows) return;
  const uint2 w = *reinterpret_cast<const uint2*>(q + r * kKv8Dim + 4 * lane);
  const float4 x = {ClampF16(WidenBf16(static_cast<uint16_t>(w.x & 0xFFFF))), ClampF16(WidenBf16(static_cast<uint16_t>(w.x >> 16))),
                    ClampF16(WidenBf16(static_cast<uint16_t>(w.y & 0xFFFF))), ClampF16(WidenBf16(static_cast<uint16_t>(w.y >> 16)))};
  const float4 h = WaveHadamard256(x, lane);
  *reinterpret_cast<uint2*>(out + r * kKv8Dim + 4 * lane) =
      uint2{PackF16(h.x * 0.0625f, h.y * 0.0625f), PackF16(h.z * 0.0625f, h.w * 0.0625f)};
}
template <int DUMMY>
__global__ __launch_bounds__(256) void PrefillImagesKv8(const ImageArgs a) {
  constexpr int D = kKv8Dim, PT = kKv8Page, CPR = D / 8;
  const Geom g = a.g;
  const Kv8Geom kg{g.n_q, g.n_kv, g.n_pages, Kv8BitsK(g.format), Kv8BitsV(g.format)};
  const int H = g.n_kv, tile = blockIdx.x, pair = blockIdx.y, s = pair / H, h = pair % H, tid = threadIdx.x;
  const int n_keys = ClampPrefix(a.prefix_len, s, a.max_prefix, a.stride, PT, a.chunk_len) + a.chunk_len;
  if (tile * kKeys >= n_keys) return;
  const int32_t* row = a.table + int64_t(s) * a.stride;
  char* kimg = a.img + (size_t(pair) * a.tiles_per_pair + tile) * TileImageBytes<D>();
  char* vimg = kimg + kKeys * D * 2;
  const int page = ClampPage(row[min(tile * kKeys / PT, a.stride - 1)], g.n_pages);  // a 64-key tile lies in one page
  for (int p = tid; p < kKeys * CPR; p += 256) {  // K: chunk = dims 8 c .. 8 c + 7 of one key
    const int key = p / CPR, c = (p % CPR) ^ (key % 16), kk = tile * kKeys + key;
    uint32_t o[4] = {0u, 0u, 0u, 0u};
    if (kk < n_keys) {
      const size_t r = size_t(page) * PT + kk % PT;
      if (kg.kb == 4) {  // the chunk's eight dims are one dword of codes, in the 32-dim group c / 4
        Kv4DecodePairs(StreamLoad(a.kv8.kq + kg.kq_row(r, h) + c), a.kv8.ks[kg.ks_row(r, h) + c / 4], 0, 4, o);
      } else {
        const uint2 w = StreamLoad(reinterpret_cast<const uint2*>(a.kv8.kq + kg.kq_row(r, h) + 2 * c));
        const uint32_t sc = a.kv8.ks[kg.ks_row(r, h) + c / 16];
        Kv8DecodeDword(w.x, sc, &o[0], &o[1]);
        Kv8DecodeDword(w.y, sc, &o[2], &o[3]);
      }
    }
    *reinterpret_cast<uint4*>(kimg + size_t(p) * 16) = uint4{o[0], o[1], o[2], o[3]};
  }
  for (int p = tid; p < D * 8; p += 256) {  // V: chunk = 4 + 4 keys of one dim
    const int dim = p / 8, c = (p % 8) ^ (dim % 8), s2 = c / 4, jg = c % 4;
    uint32_t o[4];
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      const int kk = tile * kKeys + 32 * s2 + 16 * hf + 4 * jg;  // four keys: dword (kk % 16) / 4 of their 16-key tile
      const size_t pt = size_t(page) * 16 + (kk / 16) % 16;
      const uint32_t st = a.kv8.vs[kg.vs_tile(h, pt) + dim];
      uint32_t u[2];
      if (kg.vb == 4) {  // keys (kk % 16) .. + 3 of the tile: pairs (kk % 8) / 2 and the next of dword (kk % 16) / 8
        Kv4DecodePairs(StreamLoad(a.kv8.vq + kg.vq_tile(h, pt) + size_t(dim) * 2 + (kk % 16) / 8), st, (kk % 8) / 2, 2, u);
      } else {
        const uint32_t w = StreamLoad(a.kv8.vq + kg.vq_tile(h, pt) + size_t(dim) * 4 + (kk % 16) / 4);
        Kv8DecodeDword(w, st, &u[0], &u[1]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e)  // keys at or past the end are zero in the image
        if (kk + e >= n_keys) u[e / 2] &= e % 2 ? 0x0000FFFFu : 0xFFFF0000u;
      o[2 * hf] = u[0], o[2 * hf + 1] = u[1];
    }
    *reinterpret_cast<uint4*>(vimg + size_t(p) * 16) = uint4{o[0], o[1], o[2], o[3]};
  }
}

// Maximum over the four lane groups of a wave (lanes n, n + 16, n + 32, n + 48): v_permlane16_swap exchanges the odd
// rows of one operand with the even rows of the other, v_permlane32_swap the upper half with the lower half; with both
// operands equal, the maximum of the two results is the maximum over the pair of rows (halves) in every lane.
__device__ __forceinline__ float MaxOverLaneGroups(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  const uint32_t r0 = r[0], r1 = r[1];  // (a bit cast applied to r[1] directly reads r[0] with this compiler)
  const float w = fmaxf(__builtin_bit_cast(float, r0), __builtin_bit_cast(float, r1));
  const uint32_t x = __builtin_bit_cast(uint32_t, w);
  const auto q = __builtin_amdgcn_permlane32_swap(x, x, false, false);
  const uint32_t q0 = q[0], q1 = q[1];
  return fmaxf(__builtin_bit_cast(float, q0), __builtin_bit_cast(float, q1));
}

template <bool B>
struct Constant {
  static constexpr bool value = B;
};

// s_waitcnt operand: at most n vector memory operations outstanding, the other counters unconstrained
constexpr int VmCnt(int n) { return 0x0F70 | (n & 15) | ((n >> 4) << 14); }

// Same work split as the fused kernel: 4 waves, 64 chunk positions x RB heads, RB row blocks of 16 queries per wave,
// everything transposed (keys along MFMA rows, queries along lanes). LDS holds two tile images.
template <int D, int RB, int KP = 1, int VP = 6>
__global__ __launch_bounds__(256) void PrefillAttendImg(const PrefillArgs a, const char* img, int tiles_per_pair) {
  constexpr int KS = D / 32, NDT = D / 16, kHeadsPerGroup = RB;
  constexpr int KIMG = kKeys * D * 2, TIMG = TileImageBytes<D>();
  constexpr int kCopies = TIMG / 1024 / 4;  // 1 KB wave-wide copies per wave and tile
  // How far the operand reads run ahead of the products that use them, in steps of the first product (8 matrix
  // instructions each) and in 16-dim tiles of the second (4 each). Measured: 1 and 6 (2 and 2: 3 % slower).
  static_assert(kCopies == KS + NDT / 2, "one copy per step of the first product and per two of the second");
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const int n_qt = (a.chunk_len + kQueries - 1) / kQueries, n_hp = (G + kHeadsPerGroup - 1) / kHeadsPerGroup;
  const int bid = blockIdx.x, xcd = bid % 8, local = bid / 8, per_pair = n_qt * n_hp;
  const int pair = xcd + 8 * (local / per_pair), qt = n_qt - 1 - (local % per_pair) / n_hp, hp = local % n_hp;
  if (pair >= a.n_seqs * H) return;
  const int s = pair / H, h = pair % H;
  const int tid = threadIdx.x, wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int qn = lane % 16, jg = lane / 16;
  const int prefix = ClampPrefix(a.prefix_len, s, a.max_prefix, a.stride, g.pt, a.chunk_len);
  const int q0 = qt * kQueries;
  const int n_keys = min(prefix + q0 + kQueries, prefix + a.chunk_len);
  const int n_tiles = (n_keys + kKeys - 1) / kKeys;

  // two K halves and three V halves of tile images: V(t + 2) is on its way in while V(t) and V(t + 1) are in use,
  // which gives its copies a whole tile's time to land (160 KB at D = 256: all the LDS of a CU)
  static_assert(TIMG == 2 * KIMG, "the two halves of an image have the same size");
  __shared__ __align__(1024) char lds[5][KIMG];  // [0], [1]: K halves; [2] .. [4]: V halves

  h8v qb[RB][KS];
  int qpos[RB], head[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    const int rb = RB * wave + i;
    head[i] = kHeadsPerGroup * hp + rb / 4;
    qpos[i] = q0 + 16 * (rb % 4) + qn;
    const int t = min(qpos[i], a.chunk_len - 1), hd = min(head[i], G - 1);
    const uint16_t* qp = a.q + ((size_t(s) * a.chunk_len + t) * g.n_q + size_t(h) * G + hd) * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) qb[i][ks] = QueryF16(qp + 32 * ks + 8 * jg, a.q_is_f16 != 0);
  }
  f4v o[RB][NDT];
  float m[RB];
  f4v lacc[RB];
#pragma unroll
  for (int i = 0; i < RB; ++i) {
    m[i] = kNegBig, lacc[i] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[i][dt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
  }
  const float sscale = a.scale * 1.4426950408889634f;
  // Copy j (of kCopies) of this wave's share of a tile image into the LDS buffer tile % 2: pieces j < kCopies / 2 are
  // the K half, the others the V half. Direct global-to-LDS loads: no registers, no vector instructions; through a
  // buffer resource of the pair's images (scalar base and offset, one 32-bit lane offset), which issues faster
  // than the flat form with its 64-bit address per lane (2 % of the kernel's time). The copies
  // are spread over the arithmetic, because the CU's vector memory path moves about 39 bytes per cycle (measured:
  // 26 cycles per 1 KB wave-wide load, 1700 cycles per 64 KB image) and a burst of them stalls every wave.
  const auto img_rsrc = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<char*>(img) + size_t(pair) * tiles_per_pair * TIMG, 0, 0x7fffffff, 0x00020000);
  auto copy_part = [&](int tile, int j) {
    const int c = wave + 4 * j;
    char* dst = j < kCopies / 2 ? lds[tile % 2] + c * 1024 : lds[2 + tile % 3] + (c * 1024 - KIMG);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(img_rsrc, (__attribute__((address_space(3))) void*)dst, 16, lane * 16,
                                             tile * TIMG + c * 1024, 0, 0);
  };
  // byte offsets of this lane's operand reads within an image; the XOR undoes the images' swizzle (K rows: chunk ^
  // (key % 16); V^T rows: chunk ^ (dim % 8)).
  // The chunk index (4 n + jg) ^ (qn % 8) is 4 (n ^ h) + (jg ^ l) with h = qn % 8 / 4 and l = qn % 4: per lane one
  // offset for even n and one for odd n, and everything else is a constant of the instruction.
  const int sw_l = 16 * (jg ^ (qn % 4)), sw_h = 64 * (qn % 8 / 4);
  // (K: (4 n + jg) ^ qn is 4 (n ^ qn / 4) + (jg ^ l): one offset per lane for each n % 4)
  int koff[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) koff[e] = qn * (2 * D) + sw_l + 64 * (e ^ (qn / 4));
  const int voff[2] = {qn * 128 + sw_l + sw_h, qn * 128 + sw_l - sw_h};
  auto read_k = [&](const char* buf, int ks, int kt) -> h8v {
    return *reinterpret_cast<const h8v*>(buf + koff[ks % 4] + (kt * 16 * (2 * D) + 64 * (ks & ~3)));
  };
  // One 32-dim step of S^T = K Q^T: the A operands of step ks + KP are read before the products of step ks.
  auto k_first = [&](const char* buf, h8v (&ka)[KP + 1][4]) {
#pragma unroll
    for (int ks = 0; ks < KP; ++ks)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) ka[ks][kt] = read_k(buf, ks, kt);
  };
  auto k_step = [&](const char* buf, int ks, h8v (&ka)[KP + 1][4], f4v (&st)[RB][4]) {
    if (ks + KP < KS) {
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) ka[(ks + KP) % (KP + 1)][kt] = read_k(buf, ks + KP, kt);
    }
#pragma unroll
    for (int kt = 0; kt < 4; ++kt)
#pragma unroll
      for (int i = 0; i < RB; ++i)
        st[i][kt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[ks % (KP + 1)][kt], qb[i][ks], st[i][kt], 0, 0, 0);
  };
  auto clear = [&](f4v (&st)[RB][4]) {
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) st[i][kt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
  };
  // Online softmax per query (= per lane). The reference point m of the numerators 2^(score - m) is a whole power
  // of two and is only moved when a score exceeds it by more than 2^(kBias + kSlack): moving it rescales numerators,
  // sums and accumulators by a power of two, which is exact, so moving it late changes nothing in the result, while f16
  // numerators and f32 sums have room for that factor. Rescaling is then rare (the first tile, mostly).
  auto row_max = [&](const f4v (&st)[4]) -> float {  // over the 64 keys of the tile, times the softmax scale
    float mx = fmaxf(st[0][0], st[0][1]);  // a chain of three-operand maxima
    mx = fmaxf(fmaxf(mx, st[0][2]), st[0][3]);
#pragma unroll
    for (int kt = 1; kt < 4; ++kt) mx = fmaxf(fmaxf(mx, st[kt][0]), st[kt][1]), mx = fmaxf(fmaxf(mx, st[kt][2]), st[kt][3]);
    return MaxOverLaneGroups(mx) * sscale;  // sscale > 0 is required by the entry point
  };
  auto move_reference = [&](int i, float mx) {
    if (__builtin_expect(__builtin_amdgcn_ballot_w64(mx > m[i] + (kBias + kSlack)) != 0, 0)) {
      const h8v zero = {0, 0, 0, 0, 0, 0, 0, 0};
      const float mn = mx > m[i] + (kBias + kSlack) ? __builtin_ceilf(mx) - kBias : m[i];
      const float alpha = __builtin_amdgcn_exp2f(m[i] - mn);
      m[i] = mn;
      // The rescaled accumulators go back through a matrix instruction with zero factors: that keeps them in the
      // accumulation registers on this path as on the common one (otherwise the compiler moves all of them to
      // ordinary registers and back in every tile, rescaled or not); the empty asm keeps the copy out of the
      // accumulation registers on this path.
      {
        f4v t = lacc[i];
        asm volatile("" : "+a"(t));
#pragma unroll
        for (int r = 0; r < 4; ++r) t[r] *= alpha;
        lacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zero, zero, t, 0, 0, 0);
      }
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) {
        f4v t = o[i][dt];
        asm volatile("" : "+a"(t));
#pragma unroll
        for (int r = 0; r < 4; ++r) t[r] *= alpha;
        o[i][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(zero, zero, t, 0, 0, 0);
      }
    }
  };
  // f16 numerators of row block i as B operands of the second product: [32-key step] 4 + 4 keys per lane
  auto numerators = [&](int i, const f4v (&st)[4], h8v (&pv)[2]) {
    uint32_t w[2][4];
#pragma unroll
    for (int kt = 0; kt < 4; ++kt) {
      float p[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) p[r] = __builtin_amdgcn_exp2f(__builtin_fmaf(st[kt][r], sscale, -m[i]));
      w[kt / 2][2 * (kt % 2)] = PackF16(p[0], p[1]);
      w[kt / 2][2 * (kt % 2) + 1] = PackF16(p[2], p[3]);
    }
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) pv[s2] = __builtin_bit_cast(h8v, uint4{w[s2][0], w[s2][1], w[s2][2], w[s2][3]});
  };
  // O^T += V^T P^T and the denominators; `v_tile` >= 0: the V half of that image is copied meanwhile (`always`:
  // known when compiling, which keeps the products in one scheduling region)
  auto pv_product = [&](auto always, const char* buf, const h8v (&pv)[RB][2], int v_tile) {
    // (the empty asm keeps the two lane addresses as they are: left alone, the compiler hoists voff + constant out
    // of the tile loop for every read and adds the buffer's address to each of them again)
    typedef __attribute__((address_space(3))) const char* LdsPtr;
    LdsPtr vb0 = (LdsPtr)buf + voff[0], vb1 = (LdsPtr)buf + voff[1];
    asm volatile("" : "+v"(vb0), "+v"(vb1));
    auto read_v = [&](int dt, int s2) -> h8v {
      return *reinterpret_cast<const __attribute__((address_space(3))) h8v*>((s2 ? vb1 : vb0) + (dt * 16 * 128 + 64 * s2));
    };
    h8v va[VP + 1][2];  // read VP 16-dim tiles ahead
#pragma unroll
    for (int dt = 0; dt < VP; ++dt)
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2) va[dt][s2] = read_v(dt, s2);
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
      for (int i = 0; i < RB; ++i)
        lacc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(OnesF16(), pv[i][s2], lacc[i], 0, 0, 0);
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) {
      if (dt + VP < NDT) {
#pragma unroll
        for (int s2 = 0; s2 < 2; ++s2) va[(dt + VP) % (VP + 1)][s2] = read_v(dt + VP, s2);
      }
#pragma unroll
      for (int s2 = 0; s2 < 2; ++s2)
#pragma unroll
        for (int i = 0; i < RB; ++i)
          o[i][dt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(va[dt % (VP + 1)][s2], pv[i][s2], o[i][dt], 0, 0, 0);
      if (dt % 2 == 1) {
        if (decltype(always)::value || v_tile >= 0) copy_part(v_tile, KS + dt / 2);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // Schedule. Iteration t has the scores S^T(t) in registers, K(t + 1), V(t) and V(t + 1) in LDS (the last maybe
  // still landing). It computes S^T(t + 1) on the matrix cores while the vector units turn S^T(t) into numerators
  // (one wave per SIMD: only instructions of the same wave can overlap), then V^T P^T(t); meanwhile K(t + 2) is
  // copied where K(t) was, and after it V(t + 2) where V(t - 1) was. One barrier per tile; it waits for the K copies,
  // issued half a tile earlier, and for the V copies of the iteration before, not for the ones just issued. Tiles that need the causal mask (the last one or two) and the last
  // tile take the plain path below the pipelined loop.
  const int n_full = min(n_tiles, (prefix + q0 + 1) / kKeys);  // tiles every query of the workgroup sees whole
  const int n_pipe = min(n_full, n_tiles - 1);
#pragma unroll
  for (int j = 0; j < kCopies; ++j) copy_part(0, j);
#pragma unroll
  for (int j = 0; j < kCopies; ++j) copy_part(min(1, n_tiles - 1), j);  // tile 1 (tile 0 again if there is none)
  __builtin_amdgcn_s_waitcnt(VmCnt(0));
  __syncthreads();
  f4v st[RB][4];
  clear(st);
  {
    h8v ka[KP + 1][4];
    k_first(lds[0], ka);
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      k_step(lds[0], ks, ka, st);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
  int tile = 0;
  constexpr int KA = KS / 4;  // steps of the next tile's first product that run beside the row maxima
  for (; tile < n_pipe; ++tile) {
    const char* kbuf = lds[(tile + 1) % 2];
    const int k_tile = min(tile + 2, n_tiles - 1);  // its K half goes where K(tile) was (again K(last) at the end)
    f4v sn[RB][4];
    clear(sn);
    h8v ka[KP + 1][4];
    float mx[RB];
    h8v pv[RB][2];
    k_first(kbuf, ka);
#pragma unroll
    for (int ks = 0; ks < KA; ++ks) {
      k_step(kbuf, ks, ka, sn);
      copy_part(k_tile, ks);
    }
#pragma unroll
    for (int i = 0; i < RB; ++i) mx[i] = row_max(st[i]);
    // (the compiler spreads the vector work between the matrix instructions by itself; explicit scheduling groups
    // were 3 % slower)
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int i = 0; i < RB; ++i) move_reference(i, mx[i]);
#pragma unroll
    for (int ks = KA; ks < KS; ++ks) {
      k_step(kbuf, ks, ka, sn);
      copy_part(k_tile, ks);
    }
#pragma unroll
    for (int i = 0; i < RB; ++i) numerators(i, st[i], pv[i]);
    __builtin_amdgcn_sched_barrier(0);
    pv_product(Constant<true>{}, lds[2 + tile % 3], pv, min(tile + 2, n_tiles - 1));
#pragma unroll
    for (int i = 0; i < RB; ++i)
#pragma unroll
      for (int kt = 0; kt < 4; ++kt) st[i][kt] = sn[i][kt];
    // The copies complete in the order of their issue: all but the newest kCopies / 2, the pieces of V(tile + 2),
    // have landed, this wave's pieces of K(tile + 2) and V(tile + 1) among them.
    // (A bare barrier: __syncthreads() carries a release fence, which waits for every copy in flight.)
    // The wavefront-scope fences emit nothing; they keep the compiler from moving LDS accesses across the barrier,
    // which by itself is not a memory operation to it.
    __builtin_amdgcn_s_waitcnt(VmCnt(kCopies / 2) & 0xF0FF);  // and lgkmcnt(0): this wave's LDS reads have returned
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_s_barrier();  // ... and everybody's; everybody is done with K(tile + 1) and V(tile)
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  // ---- the last tiles, one phase after the other: masked softmax, second product, then the next tile's scores
  for (; tile < n_tiles; ++tile) {
    const bool more = tile + 1 < n_tiles;
    if ((tile + 1) * kKeys > prefix + q0 + 1) {  // some key of the tile is masked for some query
#pragma unroll
      for (int i = 0; i < RB; ++i)
#pragma unroll
        for (int kt = 0; kt < 4; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            if (tile * kKeys + 16 * kt + 4 * jg + r > prefix + qpos[i]) st[i][kt][r] = kNegBig;
    }
    h8v pv[RB][2];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
      move_reference(i, row_max(st[i]));
      numerators(i, st[i], pv[i]);
    }
    pv_product(Constant<false>{}, lds[2 + tile % 3], pv, tile + 2 < n_tiles ? tile + 2 : -1);
    if (more) {
      const char* kbuf = lds[(tile + 1) % 2];
      clear(st);
      h8v ka[KP + 1][4];
      k_first(kbuf, ka);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        k_step(kbuf, ks, ka, st);
        if (tile + 2 < n_tiles) copy_part(tile + 2, ks);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __builtin_amdgcn_s_waitcnt(VmCnt(0));
    __syncthreads();
  }
  StoreRows<D, RB>(a, s, h, G, jg, o, lacc, qpos, head);
}


}  // namespace
}  // namespace yahkv

using namespace yahkv;

namespace {
int32_t TilesPerPair(int32_t max_prefix_len, int32_t chunk_len) {
  return static_cast<int32_t>((int64_t(max_prefix_len) + chunk_len + kKeys - 1) / kKeys);
}
size_t ImageBytes(const Geom& m, int32_t n_seqs, int32_t max_prefix_len, int32_t chunk_len) {
  return size_t(n_seqs) * m.n_kv * TilesPerPair(max_prefix_len, chunk_len) * (size_t(2) * kKeys * m.hd * 2);
}
}  // namespace

extern "C" size_t yahkv_prefill_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_prefix_len,
                                                int32_t chunk_len) {
  if (CheckGeometry(g) || n_seqs <= 0 || max_prefix_len < 0 || chunk_len <= 0) return 0;
  return ImageBytes(MakeGeom(*g), n_seqs, max_prefix_len, chunk_len);
}

namespace {
// Checks shared by the prefill entry points and the arguments common to their kernels.
int PreparePrefill(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                   int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs, int32_t max_prefix_len,
                   int32_t chunk_len, PrefillArgs* a) {
  if (const int st = CheckPools(g, pools)) return st;
  if (page_table == nullptr || prefix_len == nullptr) return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || chunk_len <= 0 || max_prefix_len < 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  const Geom m = MakeGeom(*g);
  if (int64_t(page_table_stride) * m.pt < chunk_len) return YAHKV_ERR_ARG;
  *a = PrefillArgs{};
  a->g = m, a->pools = MakePools(*pools), a->table = page_table, a->stride = page_table_stride;
  a->prefix_len = prefix_len, a->n_seqs = n_seqs, a->max_prefix = max_prefix_len, a->chunk_len = chunk_len;
  return YAHKV_OK;
}
int PrepareQueries(const void* q, float softmax_scale, const float* gate, void* out, int32_t out_dtype,
                   PrefillArgs* a) {
  if (q == nullptr || out == nullptr || !(softmax_scale > 0.0f)) return YAHKV_ERR_ARG;
  if (out_dtype != YAHKV_F32 && out_dtype != YAHKV_F16 && out_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(q) | reinterpret_cast<uintptr_t>(out)) & 15) return YAHKV_ERR_ARG;
  a->q = static_cast<const uint16_t*>(q), a->scale = softmax_scale, a->gate = gate, a->out = out;
  a->out_dtype = out_dtype;
  return YAHKV_OK;
}
int CheckWorkspace(const PrefillArgs& a, const void* workspace, size_t workspace_bytes) {
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 15)) return YAHKV_ERR_ARG;
  return workspace_bytes < ImageBytes(a.g, a.n_seqs, a.max_prefix, a.chunk_len) ? YAHKV_ERR_WORKSPACE : YAHKV_OK;
}
// A workgroup serves 64 chunk positions of `heads_per_group` query heads of one kv head.
dim3 AttendGrid(const PrefillArgs& a, int heads_per_group) {
  const int n_qt = (a.chunk_len + kQueries - 1) / kQueries;
  const int n_hp = (a.g.group() + heads_per_group - 1) / heads_per_group;
  const int pair_slots = (a.n_seqs * a.g.n_kv + 7) / 8 * 8;
  return dim3(static_cast<unsigned>(pair_slots) * n_qt * n_hp);
}
}  // namespace

extern "C" int yahkv_prefill_decode_tiles(const yahkv_geometry* g, const yahkv_pools* pools,
                                          const int32_t* page_table, int32_t page_table_stride,
                                          const int32_t* prefix_len, int32_t n_seqs, int32_t max_prefix_len,
                                          int32_t chunk_len, void* workspace, size_t workspace_bytes, void* stream) {
  PrefillArgs a;
  if (const int rc = PreparePrefill(g, pools, page_table, page_table_stride, prefix_len, n_seqs, max_prefix_len,
                                    chunk_len, &a))
    return rc;
  if (const int rc = CheckWorkspace(a, workspace, workspace_bytes)) return rc;
  const Geom& m = a.g;
  ImageArgs ia{};
  ia.g = m, ia.pools = a.pools, ia.table = page_table, ia.stride = page_table_stride, ia.prefix_len = prefix_len;
  ia.n_seqs = n_seqs, ia.max_prefix = max_prefix_len, ia.chunk_len = chunk_len;
  ia.img = static_cast<char*>(workspace), ia.tiles_per_pair = TilesPerPair(max_prefix_len, chunk_len);
  const dim3 igrid(static_cast<unsigned>(ia.tiles_per_pair), static_cast<unsigned>(n_seqs * m.n_kv));
  hipStream_t st = static_cast<hipStream_t>(stream);
#define YAHKV_LAUNCH_IMG(FF, DD, PP) hipLaunchKernelGGL((PrefillImages<FF, DD, PP>), igrid, dim3(256), 0, st, ia)
#define YAHKV_LAUNCH_IMG_FMT(FF)                                     \
  if (m.hd == 256 && m.pt == 64) YAHKV_LAUNCH_IMG(FF, 256, 64);         \
  else if (m.hd == 256 && m.pt == 32) YAHKV_LAUNCH_IMG(FF, 256, 32);    \
  else if (m.hd == 256) YAHKV_LAUNCH_IMG(FF, 256, 16);                  \
  else if (m.pt == 64) YAHKV_LAUNCH_IMG(FF, 128, 64);                   \
  else if (m.pt == 32) YAHKV_LAUNCH_IMG(FF, 128, 32);                   \
  else YAHKV_LAUNCH_IMG(FF, 128, 16)
  if (m.format == 8) {
    YAHKV_LAUNCH_IMG_FMT(8);
  } else {
    YAHKV_LAUNCH_IMG_FMT(4);
  }
#undef YAHKV_LAUNCH_IMG_FMT
#undef YAHKV_LAUNCH_IMG
  return LaunchStatus();
}

extern "C" int yahkv_prefill_attend_tiles(const yahkv_geometry* g, const yahkv_pools* pools,
                                          const int32_t* page_table, int32_t page_table_stride,
                                          const int32_t* prefix_len, int32_t n_seqs, int32_t max_prefix_len,
                                          int32_t chunk_len, const void* q, float softmax_scale, const float* gate,
                                          void* out, int32_t out_dtype, const void* workspace, size_t workspace_bytes,
                                          void* stream) {
  PrefillArgs a;
  if (const int rc = PreparePrefill(g, pools, page_table, page_table_stride, prefix_len, n_seqs, max_prefix_len,
                                    chunk_len, &a))
    return rc;
  if (const int rc = PrepareQueries(q, softmax_scale, gate, out, out_dtype, &a)) return rc;
  const int tiles = TilesPerPair(max_prefix_len, chunk_len);
  // the attention kernel addresses a pair's images with 32-bit offsets (checked before the workspace's size, so that
  // no size a caller claims can get such a launch through)
  if (int64_t(tiles) * (2 * kKeys * a.g.hd * 2) > 0x7fffffffLL) return YAHKV_ERR_SHAPE;
  if (const int rc = CheckWorkspace(a, workspace, workspace_bytes)) return rc;
  const char* img = static_cast<const char*>(workspace);
  hipStream_t st = static_cast<hipStream_t>(stream);
  // Three row blocks per wave (three heads per workgroup) when the GQA group is a multiple of three: each tile image
  // copied to LDS and each operand read from it then serves half as much arithmetic again. At head_dim 256 that is 504 of
  // the wave's 512 registers (192 + 96 accumulation registers for O^T and two S^T, 96 for the queries' operands), no
  // spills, and worth 2 - 3 % of the kernel's time against two row blocks.
#define YAHKV_LAUNCH_ATT(DD, RR) \
  hipLaunchKernelGGL((PrefillAttendImg<DD, RR>), AttendGrid(a, RR), dim3(256), 0, st, a, img, tiles)
  if (a.g.hd == 256 && a.g.group() % 3 == 0) YAHKV_LAUNCH_ATT(256, 3);
  else if (a.g.hd == 256) YAHKV_LAUNCH_ATT(256, 2);
  else if (a.g.group() % 3 == 0) YAHKV_LAUNCH_ATT(128, 3);
  else YAHKV_LAUNCH_ATT(128, 2);
#undef YAHKV_LAUNCH_ATT
  return LaunchStatus();
}

extern "C" int yahkv_prefill_attend(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                    int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs,
                                    int32_t max_prefix_len, int32_t chunk_len, const void* q, float softmax_scale,
                                    const float* gate, void* out, int32_t out_dtype, void* workspace,
                                    size_t workspace_bytes, void* stream) {
  if (workspace != nullptr) {
    {  // everything the second dispatch would refuse is refused here, before the first one is queued
      PrefillArgs chk;
      if (const int rc = PreparePrefill(g, pools, page_table, page_table_stride, prefix_len, n_seqs, max_prefix_len,
                                        chunk_len, &chk))
        return rc;
      if (const int rc = PrepareQueries(q, softmax_scale, gate, out, out_dtype, &chk)) return rc;
      if (int64_t(TilesPerPair(max_prefix_len, chunk_len)) * (2 * kKeys * chk.g.hd * 2) > 0x7fffffffLL) return YAHKV_ERR_SHAPE;
      if (const int rc = CheckWorkspace(chk, workspace, workspace_bytes)) return rc;
    }
    if (const int rc = yahkv_prefill_decode_tiles(g, pools, page_table, page_table_stride, prefix_len, n_seqs,
                                                  max_prefix_len, chunk_len, workspace, workspace_bytes, stream))
      return rc;
    return yahkv_prefill_attend_tiles(g, pools, page_table, page_table_stride, prefix_len, n_seqs, max_prefix_len,
                                      chunk_len, q, softmax_scale, gate, out, out_dtype, workspace, workspace_bytes,
                                      stream);
  }
  // one pass: tiles are decoded inside the attention kernel
  PrefillArgs a;
  if (const int rc = PreparePrefill(g, pools, page_table, page_table_stride, prefix_len, n_seqs, max_prefix_len,
                                    chunk_len, &a))
    return rc;
  if (const int rc = PrepareQueries(q, softmax_scale, gate, out, out_dtype, &a)) return rc;
  const Geom& m = a.g;
  const dim3 grid = AttendGrid(a, kFusedRowBlocks);
  hipStream_t st = static_cast<hipStream_t>(stream);
#define YAHKV_LAUNCH_PF(FF, DD, PP) hipLaunchKernelGGL((PrefillAttendFused<FF, DD, PP>), grid, dim3(256), 0, st, a)
#define YAHKV_LAUNCH_PF_FMT(FF)                                      \
  if (m.hd == 256 && m.pt == 64) YAHKV_LAUNCH_PF(FF, 256, 64);          \
  else if (m.hd == 256 && m.pt == 32) YAHKV_LAUNCH_PF(FF, 256, 32);     \
  else if (m.hd == 256) YAHKV_LAUNCH_PF(FF, 256, 16);                   \
  else if (m.pt == 64) YAHKV_LAUNCH_PF(FF, 128, 64);                    \
  else if (m.pt == 32) YAHKV_LAUNCH_PF(FF, 128, 32);                    \
  else YAHKV_LAUNCH_PF(FF, 128, 16)
  if (m.format == 8) {
    YAHKV_LAUNCH_PF_FMT(8);
  } else {
    YAHKV_LAUNCH_PF_FMT(4);
  }
#undef YAHKV_LAUNCH_PF_FMT
#undef YAHKV_LAUNCH_PF
  return LaunchStatus();
}


extern "C" size_t yahkv_f16_prefill_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_prefix_len,
                                                    int32_t chunk_len) {
  if (g == nullptr || g->format != YAHKV_KV_F16 || n_seqs <= 0 || max_prefix_len < 0 || chunk_len <= 0) return 0;
  yahkv_geometry gq = *g;
  gq.format = YAHKV_Q8_0;
  if (CheckGeometry(&gq)) return 0;
  return ImageBytes(MakeGeom(gq), n_seqs, max_prefix_len, chunk_len);
}

// Chunked-prefill attention over unquantized f16 pools (the pools of yahkv_f16_append; the reference's attention
// reads its 16-bit K / V pool directly, gen_attn_fa.py:1589-1595): the keys' tile images are converted from the
// pools, then the same attention kernel as for the quantized formats runs on them.
extern "C" int yahkv_f16_prefill_attend(const yahkv_geometry* g, const yahkv_f16_pools* pools,
                                        const int32_t* page_table, int32_t page_table_stride,
                                        const int32_t* prefix_len, int32_t n_seqs, int32_t max_prefix_len,
                                        int32_t chunk_len, const void* q, float softmax_scale, const float* gate,
                                        void* out, int32_t out_dtype, void* workspace, size_t workspace_bytes,
                                        void* stream) {
  if (g == nullptr) return YAHKV_ERR_ARG;
  if (g->format != YAHKV_KV_F16) return YAHKV_ERR_SHAPE;
  yahkv_geometry gq = *g;
  gq.format = YAHKV_Q8_0;  // the same limits on heads, head_dim, page size and pool
  if (const int rc = CheckGeometry(&gq)) return rc;
  if (pools == nullptr || pools->k == nullptr || pools->v == nullptr || page_table == nullptr || prefix_len == nullptr)
    return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || chunk_len <= 0 || max_prefix_len < 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(pools->k) | reinterpret_cast<uintptr_t>(pools->v)) & 15) return YAHKV_ERR_ARG;
  if (pools->k_bytes < yahkv_f16_pool_bytes(g) || pools->v_bytes < yahkv_f16_pool_bytes(g)) return YAHKV_ERR_ARG;
  PrefillArgs a{};
  a.g = MakeGeom(gq);
  if (int64_t(page_table_stride) * a.g.pt < chunk_len) return YAHKV_ERR_ARG;
  a.table = page_table, a.stride = page_table_stride, a.prefix_len = prefix_len, a.n_seqs = n_seqs;
  a.max_prefix = max_prefix_len, a.chunk_len = chunk_len;
  if (const int rc = PrepareQueries(q, softmax_scale, gate, out, out_dtype, &a)) return rc;
  const int tiles = TilesPerPair(max_prefix_len, chunk_len);
  if (int64_t(tiles) * (2 * kKeys * a.g.hd * 2) > 0x7fffffffLL) return YAHKV_ERR_SHAPE;
  if (const int rc = CheckWorkspace(a, workspace, workspace_bytes)) return rc;
  ImageArgs ia{};
  ia.g = a.g, ia.table = page_table, ia.stride = page_table_stride, ia.prefix_len = prefix_len, ia.n_seqs = n_seqs;
  ia.max_prefix = max_prefix_len, ia.chunk_len = chunk_len, ia.img = static_cast<char*>(workspace);
  ia.tiles_per_pair = tiles;
  ia.fk = static_cast<const uint16_t*>(pools->k), ia.fv = static_cast<const uint16_t*>(pools->v);
  const dim3 igrid(static_cast<unsigned>(tiles), static_cast<unsigned>(n_seqs * a.g.n_kv));
  hipStream_t st = static_cast<hipStream_t>(stream);
#define YAHKV_LAUNCH_IMG16(DD, PP) hipLaunchKernelGGL((PrefillImagesF16<DD, PP>), igrid, dim3(256), 0, st, ia)
  if (a.g.hd == 256 && a.g.pt == 64) YAHKV_LAUNCH_IMG16(256, 64);
  else if (a.g.hd == 256 && a.g.pt == 32) YAHKV_LAUNCH_IMG16(256, 32);
  else if (a.g.hd == 256) YAHKV_LAUNCH_IMG16(256, 16);
  else if (a.g.pt == 64) YAHKV_LAUNCH_IMG16(128, 64);
  else if (a.g.pt == 32) YAHKV_LAUNCH_IMG16(128, 32);
  else YAHKV_LAUNCH_IMG16(128, 16);
#undef YAHKV_LAUNCH_IMG16
  if (const int rc = LaunchStatus()) return rc;
  const char* img = static_cast<const char*>(workspace);
#define YAHKV_LAUNCH_ATT(DD, RR) \
  hipLaunchKernelGGL((PrefillAttendImg<DD, RR>), AttendGrid(a, RR), dim3(256), 0, st, a, img, tiles)
  if (a.g.hd == 256 && a.g.group() % 3 == 0) YAHKV_LAUNCH_ATT(256, 3);
  else if (a.g.hd == 256) YAHKV_LAUNCH_ATT(256, 2);
  else if (a.g.group() % 3 == 0) YAHKV_LAUNCH_ATT(128, 3);
  else YAHKV_LAUNCH_ATT(128, 2);
#undef YAHKV_LAUNCH_ATT
  return LaunchStatus();
}

extern "C" size_t yahkv_kv8_prefill_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_prefix_len,
                                                    int32_t chunk_len) {
  if (CheckKv8Geometry(g) || n_seqs <= 0 || max_prefix_len < 0 || chunk_len <= 0) return 0;
  // 4-bit K: the chunk's rotated queries (f16) lie behind the images
  const size_t rotated = Kv8BitsK(g->format) == 4 ? size_t(n_seqs) * chunk_len * g->n_q_heads * kKv8Dim * 2 : 0;
  return ImageBytes(MakeGeom(*g), n_seqs, max_prefix_len, chunk_len) + rotated;
}

// Chunked-prefill attention over kv8a16 pools: the keys' f16 tile images are decoded from the pools with the reference's
// own prefill-side decode, then the same attention kernel as for the other formats runs on them.
extern "C" int yahkv_kv8_prefill_attend(const yahkv_geometry* g, const yahkv_kv8_pools* pools,
                                        const int32_t* page_table, int32_t page_table_stride,
                                        const int32_t* prefix_len, int32_t n_seqs, int32_t max_prefix_len,
                                        int32_t chunk_len, const void* q, float softmax_scale, const float* gate,
                                        void* out, int32_t out_dtype, void* workspace, size_t workspace_bytes,
                                        void* stream) {
  if (const int rc = CheckKv8Pools(g, pools)) return rc;
  if (page_table == nullptr || prefix_len == nullptr) return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || chunk_len <= 0 || max_prefix_len < 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  PrefillArgs a{};
  a.g = MakeGeom(*g);
  if (int64_t(page_table_stride) * a.g.pt < chunk_len) return YAHKV_ERR_ARG;
  a.table = page_table, a.stride = page_table_stride, a.prefix_len = prefix_len, a.n_seqs = n_seqs;
  a.max_prefix = max_prefix_len, a.chunk_len = chunk_len;
  if (const int rc = PrepareQueries(q, softmax_scale, gate, out, out_dtype, &a)) return rc;
  const int tiles = TilesPerPair(max_prefix_len, chunk_len);
  if (int64_t(tiles) * (2 * kKeys * a.g.hd * 2) > 0x7fffffffLL) return YAHKV_ERR_SHAPE;
  if (const int rc = CheckWorkspace(a, workspace, workspace_bytes)) return rc;
  if (workspace_bytes < yahkv_kv8_prefill_workspace_bytes(g, n_seqs, max_prefix_len, chunk_len)) return YAHKV_ERR_WORKSPACE;
  ImageArgs ia{};
  ia.g = a.g, ia.table = page_table, ia.stride = page_table_stride, ia.prefix_len = prefix_len, ia.n_seqs = n_seqs;
  ia.max_prefix = max_prefix_len, ia.chunk_len = chunk_len, ia.img = static_cast<char*>(workspace);
  ia.tiles_per_pair = tiles, ia.kv8 = MakeKv8Pools(*pools);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (Kv8BitsK(g->format) == 4) {
    uint16_t* rotated = reinterpret_cast<uint16_t*>(static_cast<char*>(workspace) + ImageBytes(a.g, n_seqs, max_prefix_len, chunk_len));
    const int64_t rows = int64_t(n_seqs) * chunk_len * a.g.n_q;
    hipLaunchKernelGGL(Kv4RotateQ, dim3(static_cast<unsigned>((rows + 3) / 4)), dim3(256), 0, st, a.q, rotated, rows);
    if (const int rc = LaunchStatus()) return rc;
    a.q = rotated, a.q_is_f16 = 1;
  }
  hipLaunchKernelGGL(PrefillImagesKv8<0>, dim3(static_cast<unsigned>(tiles), static_cast<unsigned>(n_seqs * a.g.n_kv)),
                     dim3(256), 0, st, ia);
  if (const int rc = LaunchStatus()) return rc;
  if (a.g.group() % 3 == 0)
    hipLaunchKernelGGL((PrefillAttendImg<256, 3>), AttendGrid(a, 3), dim3(256), 0, st, a, static_cast<const char*>(workspace), tiles);
  else
    hipLaunchKernelGGL((PrefillAttendImg<256, 2>), AttendGrid(a, 2), dim3(256), 0, st, a, static_cast<const char*>(workspace), tiles);
  return LaunchStatus();
}
