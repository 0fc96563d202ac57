// Paged GQA decode attention over kv8a16 pools (the reference's own KV format, see kv8.hpp): split-K over the closed
// 16-key V tiles, then a merge that also takes the keys of the open tile and, in the step form, appends the step's token.
//
// Follows yah_dattn_part_q + yah_dattn_reduce (engine/gpu/loom/tools/gen_decode_attn.py:576-1040, 338-411): K of every
// key from codes, `(u - 128) * S / 256` per 128-dim half; V of every tile before the newest from codes,
// `u * (S / 256) + (S + C')`; the newest tile from the open f16 tile; keys at or past the length masked. The cut of the
// work (stream-K over a line of 64-key tiles, one 8-wave workgroup per CU) is the one of decode.hip, shared through
// decode_cut.hpp; what differs is what a wave does with a tile:
//   K rows lie [token][kv head][256 bytes], so the 32 keys a score instruction wants (one key per lane) are 256-byte
//      pieces 1 KB apart. They are copied to the wave's LDS slot by `buffer_load ... lds` with each row's 256 bytes
//      across 16 lanes (whole cache lines per wave instruction), 16-byte chunks XOR-swizzled by row so that the
//      operand reads (lane = key) meet no bank conflicts. Scores run on v_mfma_f32_32x32x16_f16 over the codes with
//      their f16 constant still on (0x6400 | u = 1024 + u); per 128-dim half and head the constant's share,
//      1152 * sum(q), comes off the f32 sum before the half's scale goes on, so the products are exact.
//   V tiles lie [kv head][tile][dim][16 keys]: a lane's 16-byte load is one dim's 16 keys of one tile, which with four
//      tiles across the four lane groups is the operand shape of v_mfma_f32_16x16x32_f16. Codes become f16
//      1 + u / 256 by a shift and a mask (what the byte order (k0, k2, k1, k3) is for, gen_kvq.py:480-483) and one
//      packed f16 fma with the (tile, dim) stats gives the value (the reference's prefill-side decode; its decode side
//      does the same in f32). P is rounded to f16 as in decode.hip.
#include <algorithm>
#include <cstdint>

#include "decode_cut.hpp"
#include "kv8.hpp"
#include "quant.hpp"

namespace yahkv {
namespace {

// ---- the split-K kernel ---------------------------------------------------------------------------------------------
// KB / VB: bits of the K and of the V codes (8: kv8a16, 4: kv4a16; see kv8.hpp). What differs with 4 bits:
//   K rows are 128 bytes (eight 16-byte chunks = the eight 32-dim groups of a head); a key's dword (eight dims) becomes
//      the f16 values 1 + u / 16 by four shifts and masks, the two matrix instructions of a group sum (1 + u / 16) q'
//      over its 32 dims, and with the group's pair (S, C) = (16 s, lo - 16 s) the group's share of the score is
//      S * sum + C * (sum of the group's q'): the format's own `(1 + u / 16) * S + C`, exact in f32. q' = H256 q / 16
//      is made by each wave when it starts on a pair (f32 butterflies in the reference's order, then f16).
//   V codes are 8 bytes per (dim, tile); a dword's nibbles are keys (0, 2, 4, 6, 1, 3, 5, 7) of its eight, so the same
//      shifts and masks give the key pairs in order, and one packed f16 fma with (16 s, c - 23 s) the values.
template <int KB, int VB>
__global__ __launch_bounds__(64 * kWavesPerGroup) __attribute__((amdgpu_waves_per_eu(2, 2)))
void Kv8Part(const DecodeArgs a, const Kv8Pools pools) {
  constexpr int D = kKv8Dim, NT = D / 16;
  constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const size_t tiles16 = size_t(g.n_pages) * 16;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
  const int n32 = lane % 32, half = lane / 32;
  const int n16 = lane % 16, kg = lane / 16;

  // Query A-operands [step m of 16][lane half][head row][8 dims]: step m = 2 j + sub covers, in lane half hf, the 8
  // bytes `sub` of the 16-byte chunk 2 j + hf of a key's row: dims 16 (2 j + hf) + 8 sub + (0, 2, 1, 3, 4, 6, 5, 7).
  __shared__ __align__(16) _Float16 lq_all[kWavesPerGroup][16][2][8][8];
  __shared__ __align__(16) float lcorr_all[kWavesPerGroup][KB == 4 ? 8 : 2][8];
  __shared__ __align__(16) _Float16 lp_all[kWavesPerGroup][kMaxGroup][kTile];
  __shared__ __align__(16) uint8_t lk_all[kWavesPerGroup][32 * (KB == 4 ? 128 : 256)];  // 32 key rows, chunks swizzled by row
  __shared__ int next_tile;
  __shared__ int progress[kWavesPerGroup];  // tiles each wave is through with (fixed pattern only)
  __shared__ int wave_sum[kWavesPerGroup][2];
  __shared__ int4 chunk_rec;
  __shared__ long long chunk_tiles[4];
  auto& lq = lq_all[wave];
  auto& lcorr = lcorr_all[wave];
  auto& lp = lp_all[wave];
  auto& lk = lk_all[wave];

  if (a.stamps != nullptr && threadIdx.x == 0) a.stamps[blockIdx.x] = wall_clock64();
  const int chunk_id = static_cast<int>(blockIdx.x);
  bool any_empty = false;
  const int4 rec_v = a.n_seqs <= 64 ? ChunkRecordWave(a, chunk_id, wave, lane, &chunk_rec, chunk_tiles, &any_empty)
                                    : ChunkRecord<64 * kWavesPerGroup>(a, chunk_id, wave_sum, &chunk_rec, chunk_tiles, &any_empty);
  // (the record is the same in every lane: scalar registers for it and for everything derived from it)
  const int4 rec = {__builtin_amdgcn_readfirstlane(rec_v.x), __builtin_amdgcn_readfirstlane(rec_v.y),
                    __builtin_amdgcn_readfirstlane(rec_v.z), __builtin_amdgcn_readfirstlane(rec_v.w)};
  if (rec.x < 0) return;
  const int chunk_n = rec.w;
  // The line's items: tiles of a (sequence, kv head) pair, or, with a.tile_mult = H, the H kv heads of a sequence's tiles
  // one after the other. There wave w of the fixed pattern keeps its kv head as long as it stays with a sequence (its
  // items are eight apart and H divides eight), and the waves of a workgroup take the heads of a tile side by side:
  // the row of `ks` that holds a token's scale pairs of all heads is fetched once instead of once per head.
  const int lg_mult = a.tile_mult > 1 ? __builtin_ctz(static_cast<unsigned>(a.tile_mult)) : 0;
  const bool fixed_pattern = a.deterministic || chunk_n <= kWavesPerGroup || lg_mult > 0;  // (one tile per wave: no hand-out)
  if (!fixed_pattern) {
    if (threadIdx.x == 0) next_tile = 0;
    __syncthreads();
  }
  int my_next = wave;
  // (see decode.hip: with a fixed pattern the two waves of a SIMD pace each other through their priorities)
  int done_tiles = 0;
  if (lane == 0) progress[wave] = 0;
  auto pace = [&]() {
    if (!fixed_pattern) return;
    ++done_tiles;
    int other = 0;
    if (lane == 0) {
      __hip_atomic_store(&progress[wave], done_tiles, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
      other = __hip_atomic_load(&progress[wave ^ 4], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
    other = __builtin_amdgcn_readfirstlane(other);
    if (done_tiles < other) __builtin_amdgcn_s_setprio(2);
    else __builtin_amdgcn_s_setprio(0);
  };
  auto take = [&]() -> int {
    if (fixed_pattern) {
      const int v = my_next;
      my_next += kWavesPerGroup;
      return v;
    }
    int v = 0;
    if (lane == 0) v = __hip_atomic_fetch_add(&next_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return __builtin_amdgcn_readfirstlane(v);
  };

  uint2 ksc;       // this lane's key: the two halves' scale pairs
  uint4 ksc4[2];   // 4-bit K: the eight groups' pairs
  uint4 vb[VB == 4 ? 1 : NT / 2];  // 16 keys of this lane's dim in this lane group's tile (one half of the dims at a time)
  uint2 vb4[VB == 4 ? NT / 2 : 1];
  uint32_t vst[NT / 2];
  float m[4], lsum[4], sc[2][4];
  f4v o[NT];
  const float qk_scale = a.scale * kLog2e;
  const int prow = n16 < 4 ? n16 : (n16 >= 8 && n16 < 12 ? n16 - 4 : 0);

  PairCursor cur = FirstPair(a, rec);
  int head = 0;  // the kv head of the wave's current items
  const int32_t* row = nullptr;
  typedef const int32_t __attribute__((address_space(4))) * ConstRow;
  // a 64-key tile lies inside one 256-token page
  auto load_page = [&](int tile) -> int {
    const ConstRow crow = (ConstRow)(reinterpret_cast<uintptr_t>(row));
    return ClampPage(crow[min(tile / 4, a.stride - 1)], g.n_pages);
  };
  // A pair's query entries of this lane, four pieces of eight dims of head row `rw` (first dim of piece e: dim0(e)): all
  // four asked for together, under one branch on the type. With the type looked at load by load each piece's load sat in
  // a branch of its own and went out when the one before had come back. A row past the group's asks for the last one;
  // the caller zeroes it.
  auto load_queries = [&](RawQ8 (&rq)[4], auto dim0, int rw) {
    const size_t row = (size_t(cur.s) * g.n_q + size_t(head) * G + min(rw, G - 1)) * D;
    if (a.q_dtype == YAHKV_F32) {
#pragma unroll
      for (int e = 0; e < 4; ++e) rq[e] = LoadRawQ8(a.q, row + dim0(e), YAHKV_F32);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) rq[e] = LoadRawQ8(a.q, row + dim0(e), YAHKV_F16);  // (16 bytes for bf16 as well)
    }
  };
  // K: the 32 rows of half tile tt to the LDS slot, four rows per instruction; lane l of instruction i carries chunk
  // (l % 16) ^ (row % 16) of row 4 i + l / 16 to LDS position 1024 i + 16 l
  // `live` false: a load whose result nobody uses (it keeps the count of loads in flight the same on every path):
  // every lane reads the start of the piece, a few lines for the whole wave instead of the piece itself.
  auto load_k = [&](int tile, int tt, int page, bool live = true) {
    const size_t row0 = size_t(page) * kKv8Page + (tile % 4) * kTile + 32 * tt;
    if constexpr (KB == 4) {
      // eight rows per instruction; lane l of instruction i carries chunk (l % 8) ^ (row % 8) of row 8 i + l / 8
      const auto rk4 = __builtin_amdgcn_make_buffer_rsrc(
          reinterpret_cast<uint8_t*>(pools.kq) + (row0 * H + head) * 128, 0, 0x7fffffff, 0x00020000);
      const uint32_t r = lane / 8, c = lane % 8;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t rr = 8 * i + r;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rk4, (__attribute__((address_space(3))) void*)(&lk[i * 1024]), 16,
                                                 live ? rr * (H * 128) + ((c ^ (rr & 7)) << 4) : 0u, 0, 0, kStreamed);
      }
      const uint32_t* sp4 = pools.ks + ((row0 + (live ? n32 : 0)) * H + head) * 8;
      // (plain loads: the row's other quarters are wanted by the waves next to this one, and a streaming read leaves
      // nothing in the L2 for them)
      ksc4[0] = *reinterpret_cast<const uint4*>(sp4);
      ksc4[1] = *reinterpret_cast<const uint4*>(sp4 + 4);
    } else {
      const auto rk = __builtin_amdgcn_make_buffer_rsrc(
          reinterpret_cast<uint8_t*>(pools.kq) + (row0 * H + head) * 256, 0, 0x7fffffff, 0x00020000);
      const uint32_t r = lane / 16, c = lane % 16;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t rr = 4 * i + r;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rk, (__attribute__((address_space(3))) void*)(&lk[i * 1024]), 16,
                                                 live ? rr * (H * 256) + ((c ^ (rr & 15)) << 4) : 0u, 0, 0, kStreamed);
      }
      const uint32_t* sp = pools.ks + ((row0 + (live ? n32 : 0)) * H + head) * 2;
      ksc = *reinterpret_cast<const uint2*>(sp);  // (a plain load, as for the 4-bit rows)
    }
  };
  auto fetch_v = [&](int tile, int hf, int page, bool live = true) {
    const size_t pt = size_t(page) * 16 + (tile % 4) * 4 + (live ? kg : 0);
    const int dim = 128 * hf + (live ? n16 : 0);
    const uint32_t* vp = pools.vq + ((size_t(head) * tiles16 + pt) * 256 + dim) * (VB == 4 ? 2 : 4);
    const uint32_t* sp = pools.vs + (size_t(head) * tiles16 + pt) * 256 + dim;
    if constexpr (VB == 4) {
#pragma unroll
      for (int j = 0; j < NT / 2; ++j) vb4[j] = StreamLoad(reinterpret_cast<const uint2*>(vp + 32 * j));
    } else {
#pragma unroll
      for (int j = 0; j < NT / 2; ++j) vb[j] = StreamLoad(reinterpret_cast<const uint4*>(vp + 64 * j));
    }
#pragma unroll
    for (int j = 0; j < NT / 2; ++j) vst[j] = StreamLoad(sp + 16 * j);
  };
  // scores of the 32 keys in the LDS slot against all heads: the two 128-dim halves are two accumulator chains
  // `(x & mask) | one` is one instruction (v_and_or_b32) only if neither constant is a literal, which that encoding does
  // not take: the mask is handed to the compiler in a scalar register and the f16 pair (1.0, 1.0) in a vector register,
  // both behind an empty asm it cannot see through (with literals it emits an `and` and an `or`: a third more
  // instructions for every pair of codes).
  // (8-bit codes keep the literals: that kernel is bound by memory, and the register this takes costs it spills.)
  uint32_t one2 = 0x3c003c00u, mask4 = 0x03c003c0u;
  if constexpr (KB == 4 || VB == 4) {
    asm volatile("" : "+v"(one2));
    asm volatile("" : "+s"(mask4));
  }
  // a dword of eight 4-bit codes (dims 2 j / 2 j + 1 at bits 4 j / 16 + 4 j) as the f16 values 1 + u / 16 in dim order
  auto nibbles_f16 = [&](uint32_t w) -> h8v {
    const uint4 k = {((w << 6) & mask4) | one2, ((w << 2) & mask4) | one2, ((w >> 2) & mask4) | one2, ((w >> 6) & mask4) | one2};
    return __builtin_bit_cast(h8v, k);
  };
  auto scores = [&](int tt) {
    f16v c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0;
    if constexpr (KB == 4) {
      // group c = chunk c of the key's row; lane half hf holds dwords 2 hf, 2 hf + 1 of it: steps 2 c and 2 c + 1
      const uint32_t pr[8] = {ksc4[0].x, ksc4[0].y, ksc4[0].z, ksc4[0].w, ksc4[1].x, ksc4[1].y, ksc4[1].z, ksc4[1].w};
      float acc[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
      for (int c = 0; c < 8; c += 2) {
        const uint2 w0 = *reinterpret_cast<const uint2*>(&lk[n32 * 128 + ((c ^ (n32 & 7)) << 4) + 8 * half]);
        const uint2 w1 = *reinterpret_cast<const uint2*>(&lk[n32 * 128 + (((c + 1) ^ (n32 & 7)) << 4) + 8 * half]);
        const h8v qa0 = *reinterpret_cast<const h8v*>(&lq[2 * c][half][n32 % 8][0]);
        const h8v qa1 = *reinterpret_cast<const h8v*>(&lq[2 * c + 1][half][n32 % 8][0]);
        const h8v qb0 = *reinterpret_cast<const h8v*>(&lq[2 * c + 2][half][n32 % 8][0]);
        const h8v qb1 = *reinterpret_cast<const h8v*>(&lq[2 * c + 3][half][n32 % 8][0]);
        const f16v z = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        f16v g0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa0, nibbles_f16(w0.x), z, 0, 0, 0);
        f16v g1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb0, nibbles_f16(w1.x), z, 0, 0, 0);
        g0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa1, nibbles_f16(w0.y), g0, 0, 0, 0);
        g1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb1, nibbles_f16(w1.y), g1, 0, 0, 0);
        const float4 s0 = *reinterpret_cast<const float4*>(&lcorr[c][4 * half]);
        const float4 s1 = *reinterpret_cast<const float4*>(&lcorr[c + 1][4 * half]);
        const float S0 = WidenF16(static_cast<uint16_t>(pr[c] & 0xFFFF)), C0 = WidenF16(static_cast<uint16_t>(pr[c] >> 16));
        const float S1 = WidenF16(static_cast<uint16_t>(pr[c + 1] & 0xFFFF)), C1 = WidenF16(static_cast<uint16_t>(pr[c + 1] >> 16));
        const float q0[4] = {s0.x, s0.y, s0.z, s0.w}, q1[4] = {s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          acc[r] = __builtin_fmaf(S0, g0[r], __builtin_fmaf(C0, q0[r], acc[r]));
          acc[r] = __builtin_fmaf(S1, g1[r], __builtin_fmaf(C1, q1[r], acc[r]));
        }
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) sc[tt][r] = acc[r] * qk_scale;
      return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint4 w0 = *reinterpret_cast<const uint4*>(&lk[n32 * 256 + (((2 * j + half) ^ (n32 & 15)) << 4)]);
      const uint4 w1 = *reinterpret_cast<const uint4*>(&lk[n32 * 256 + (((2 * (j + 4) + half) ^ (n32 & 15)) << 4)]);
      const h8v qa0 = *reinterpret_cast<const h8v*>(&lq[2 * j][half][n32 % 8][0]);
      const h8v qa1 = *reinterpret_cast<const h8v*>(&lq[2 * j + 1][half][n32 % 8][0]);
      const h8v qb0 = *reinterpret_cast<const h8v*>(&lq[2 * (j + 4)][half][n32 % 8][0]);
      const h8v qb1 = *reinterpret_cast<const h8v*>(&lq[2 * (j + 4) + 1][half][n32 % 8][0]);
      const uint4 ka = {__builtin_amdgcn_perm(0x64646464u, w0.x, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w0.x, 0x04030402u),
                        __builtin_amdgcn_perm(0x64646464u, w0.y, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w0.y, 0x04030402u)};
      const uint4 kb = {__builtin_amdgcn_perm(0x64646464u, w0.z, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w0.z, 0x04030402u),
                        __builtin_amdgcn_perm(0x64646464u, w0.w, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w0.w, 0x04030402u)};
      const uint4 kc = {__builtin_amdgcn_perm(0x64646464u, w1.x, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w1.x, 0x04030402u),
                        __builtin_amdgcn_perm(0x64646464u, w1.y, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w1.y, 0x04030402u)};
      const uint4 kd = {__builtin_amdgcn_perm(0x64646464u, w1.z, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w1.z, 0x04030402u),
                        __builtin_amdgcn_perm(0x64646464u, w1.w, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, w1.w, 0x04030402u)};
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa0, __builtin_bit_cast(h8v, ka), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb0, __builtin_bit_cast(h8v, kc), c1, 0, 0, 0);
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa1, __builtin_bit_cast(h8v, kb), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb1, __builtin_bit_cast(h8v, kd), c1, 0, 0, 0);
    }
    const float4 k0 = *reinterpret_cast<const float4*>(&lcorr[0][4 * half]);
    const float4 k1 = *reinterpret_cast<const float4*>(&lcorr[1][4 * half]);
    const float kc0[4] = {k0.x, k0.y, k0.z, k0.w}, kc1[4] = {k1.x, k1.y, k1.z, k1.w};
    const float d0 = WidenF16(static_cast<uint16_t>(ksc.x & 0xFFFF)) * (qk_scale * 0.00390625f);
    const float d1 = WidenF16(static_cast<uint16_t>(ksc.y & 0xFFFF)) * (qk_scale * 0.00390625f);
#pragma unroll
    for (int r = 0; r < 4; ++r) sc[tt][r] = __builtin_fmaf(c1[r] - kc1[r], d1, (c0[r] - kc0[r]) * d0);
  };
  // P.V for one half of the dims, from vb, vst and lp; tiles at or past `live16` (the pair's closed tiles) count zero
  auto pv = [&](int tile, int hf, int live16) {
    const h8v pa0 = *reinterpret_cast<const h8v*>(&lp[prow][16 * kg]);
    const h8v pa1 = *reinterpret_cast<const h8v*>(&lp[prow][16 * kg + 8]);
    const bool dead = tile * 4 + kg >= live16;
#pragma unroll
    for (int j = 0; j < NT / 2; ++j) {
      const uint32_t st = dead ? 0u : vst[j];
      const h2v sp = __builtin_bit_cast(h2v, st);
      const h2v S2 = {sp[0], sp[0]}, C2 = {sp[1], sp[1]};
      if constexpr (VB == 4) {
        // dword w holds keys 8 w + (0, 2, 4, 6 | 1, 3, 5, 7): the pairs (2 p, 2 p + 1) sit 16 bits apart
        const h8v u0 = nibbles_f16(vb4[j].x), u1 = nibbles_f16(vb4[j].y);
        const h8v S8 = {sp[0], sp[0], sp[0], sp[0], sp[0], sp[0], sp[0], sp[0]};
        const h8v C8 = {sp[1], sp[1], sp[1], sp[1], sp[1], sp[1], sp[1], sp[1]};
        const h8v v0 = __builtin_elementwise_fma(u0, S8, C8), v1 = __builtin_elementwise_fma(u1, S8, C8);
        const int nt = hf * (NT / 2) + j;
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa0, v0, o[nt], 0, 0, 0);
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa1, v1, o[nt], 0, 0, 0);
        continue;
      }
      const uint32_t w[4] = {vb[j].x, vb[j].y, vb[j].z, vb[j].w};
      h2v f[8];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        f[2 * i] = __builtin_bit_cast(h2v, ((w[i] << 2) & 0x03fc03fcu) | 0x3c003c00u);      // keys 4 i, 4 i + 1
        f[2 * i + 1] = __builtin_bit_cast(h2v, ((w[i] >> 6) & 0x03fc03fcu) | 0x3c003c00u);  // keys 4 i + 2, 4 i + 3
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) f[i] = __builtin_elementwise_fma(f[i], S2, C2);
      const h8v v0 = {f[0][0], f[0][1], f[1][0], f[1][1], f[2][0], f[2][1], f[3][0], f[3][1]};
      const h8v v1 = {f[4][0], f[4][1], f[5][0], f[5][1], f[6][0], f[6][1], f[7][0], f[7][1]};
      const int nt = hf * (NT / 2) + j;
      o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa0, v0, o[nt], 0, 0, 0);
      o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa1, v1, o[nt], 0, 0, 0);
    }
  };
  // partial of (this chunk, this wave, the current sequence, kv head h)
  // (chunk + pair counts a wave's places along the line without collisions as long as pairs follow each other on it;
  // with a sequence as the pair, every kv head has a row of places of its own)
  auto part_of = [&](int h) -> size_t {
    if (lg_mult > 0) return ((size_t(h) * (a.n_chunks + a.n_seqs) + chunk_id + cur.s) * a.wpc + wave) * G;
    return ((size_t(chunk_id) + size_t(cur.s) * H + h) * a.wpc + wave) * G;
  };
  auto empty_at = [&](int h) {
    if (lane < G) StoreDevice2(DeviceBuffer(a.ml + part_of(h) * 2), lane * 8, kNegMax, 0.0f);
  };
  // (with the heads of a tile dealt to the waves, a wave's partial belongs to one head of the sequence; the merge of
  // another head finds this wave's place for that head empty)
  auto leave_empty = [&]() {
    if (lg_mult == 0) return empty_at(cur.h);
    for (int h = 0; h < H; ++h) empty_at(h);
  };
  auto leave_partial = [&]() {
    if (lg_mult > 0)
      for (int h = 0; h < H; ++h)
        if (h != head) empty_at(h);
    const size_t part = part_of(lg_mult > 0 ? head : cur.h);
    const auto rml = DeviceBuffer(a.ml + part * 2), racc = DeviceBuffer(a.acc + part * D);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float l = HalfSum32(lsum[r]);
      const int head = 4 * half + r;
      if (n32 == 0 && head < G) StoreDevice2(rml, head * 8, m[r] * kLn2, l);
    }
    if (kg == 0 || kg == 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int head = 2 * kg + r;
        if (head < G) {
#pragma unroll
          for (int nt = 0; nt < NT; ++nt) StoreDevice(racc, (head * D + 16 * nt + n16) * 4, o[nt][r]);
        }
      }
    }
  };

  int idx = take();
  bool worked = false;
  while (true) {
    bool more = idx < chunk_n;
    while (more && idx >= cur.base + cur.n) {
      if (!worked) leave_empty();
      worked = false;
      more = NextPair(a, chunk_n, &cur);
    }
    if (!more) break;
    // ---- first tile of this wave in the pair: query operands, the constants' shares, empty state, first loads
    row = a.table + int64_t(cur.s) * a.stride;
    const int live16 = cur.len / 16;  // closed 16-key tiles of the pair (cur.len is a multiple of 16)
    const int item = cur.first + (idx - cur.base);
    head = lg_mult > 0 ? item & (a.tile_mult - 1) : cur.h;
    int tile = item >> lg_mult;
    int pgc = load_page(tile), pgn;
    load_k(tile, 0, pgc);
    fetch_v(tile, 1, pgc, false);  // not used: keeps the count of loads in flight at the loop's head the same on every pass
    if constexpr (KB == 4) {
      // Entry e of this lane: step mm = lane / 16 + 4 e, lane half hf = (lane / 8) % 2, head row rw = lane % 8, the eight
      // dims 32 (mm / 2) + 8 (2 hf + mm % 2) + [0, 8) in their natural order. H256 over a head's 256 dims, stages in the
      // reference's order: dims 1, 2, 4 apart inside an entry; 8 apart = lane ^ 16, 16 = lane ^ 8, 32 = lane ^ 32;
      // 64 and 128 apart = entries e ^ 1 and e ^ 2.
#pragma clang fp contract(off)
      const int rw = lane % 8, hf = (lane / 8) % 2;
      float x[4][8];
      RawQ8 rq[4];
      load_queries(rq, [&](int e) {
        const int mm = lane / 16 + 4 * e;
        return 32 * (mm / 2) + 8 * (2 * hf + mm % 2);
      }, rw);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        h8v qv = ConvertQ8(rq[e], a.q_dtype);
        if (rw >= G) qv = h8v{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 8; ++k) x[e][k] = static_cast<float>(qv[k]);
#pragma unroll
        for (int st = 1; st < 8; st <<= 1)
#pragma unroll
          for (int k = 0; k < 8; ++k)
            if (!(k & st)) {
              const float lo = x[e][k], up = x[e][k | st];
              x[e][k] = lo + up, x[e][k | st] = lo - up;
            }
      }
      auto cross = [&](int xm) {
        const bool upper = (lane & xm) != 0;
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int k = 0; k < 8; ++k) {
            const float o2 = __shfl_xor(x[e][k], xm, 64);
            x[e][k] = upper ? o2 - x[e][k] : x[e][k] + o2;
          }
      };
      cross(16), cross(8), cross(32);
#pragma unroll
      for (int st = 1; st < 4; st <<= 1)
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (!(e & st))
#pragma unroll
            for (int k = 0; k < 8; ++k) {
              const float lo = x[e][k], up = x[e | st][k];
              x[e][k] = lo + up, x[e | st][k] = lo - up;
            }
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int mm = lane / 16 + 4 * e;
        h8v qs;
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
          qs[k] = static_cast<_Float16>(x[e][k] * 0.0625f);
          t += static_cast<float>(qs[k]);
        }
        *reinterpret_cast<h8v*>(&lq[mm][hf][rw][0]) = qs;
        // the group's sum of q': its four entries sit in the lanes that differ in bits 3 and 4
        t += __shfl_xor(t, 8, 64), t += __shfl_xor(t, 16, 64);
        if ((lane & 24) == 0) lcorr[2 * e + lane / 32][rw] = t;
      }
    } else {
      float hsum[2] = {0.0f, 0.0f};  // per (128-dim half, head row lane % 8): this lane's share
      // entry i = lane + 64 e: step m = i / 16, lane half hf = (i / 8) % 2, head row rw = i % 8
      RawQ8 rq[4];
      load_queries(rq, [&](int e) {
        const int i = lane + 64 * e, mm = i / 16, hf = (i / 8) % 2;
        return 16 * (2 * (mm / 2) + hf) + 8 * (mm % 2);
      }, lane % 8);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int i = lane + 64 * e, mm = i / 16, hf = (i / 8) % 2, rw = i % 8;
        h8v qv = ConvertQ8(rq[e], a.q_dtype);
        if (rw >= G) qv = h8v{0, 0, 0, 0, 0, 0, 0, 0};
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) t += static_cast<float>(qv[k]);
        hsum[mm / 8] += t;  // e = 0, 1: steps 0-7 (dims 0-127); e = 2, 3: steps 8-15
        const h8v qs = {qv[0], qv[2], qv[1], qv[3], qv[4], qv[6], qv[5], qv[7]};  // the codes' byte order
        *reinterpret_cast<h8v*>(&lq[mm][hf][rw][0]) = qs;
      }
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        float t = hsum[hh] * 1152.0f;
        t += __shfl_xor(t, 8, 64), t += __shfl_xor(t, 16, 64), t += __shfl_xor(t, 32, 64);
        if (lane < 8) lcorr[hh][lane] = t;
      }
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) m[r] = kNegMax, lsum[r] = 0.0f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) o[nt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    worked = true;
    bool first = true;
    int ptile = tile;
    while (true) {
      const int nidx = take();
      const bool has_next = nidx < cur.base + cur.n;
      const int ntile = (cur.first + (nidx - cur.base)) >> lg_mult;
      pgn = load_page(has_next ? ntile : tile);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      scores(0);
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the slot has been read before it is filled again
      __builtin_amdgcn_sched_barrier(0);
      load_k(tile, 1, pgc);
      if (!first) pv(ptile, 1, live16);
      fetch_v(tile, 0, pgc);
      first = false;
      scores(1);
      __builtin_amdgcn_s_waitcnt(0xC07F);
      __builtin_amdgcn_sched_barrier(0);
      load_k(has_next ? ntile : tile, 0, pgn, has_next);
      float alpha[4];
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        const bool valid = tile * kTile + 32 * tt + n32 < cur.len;
#pragma unroll
        for (int r = 0; r < 4; ++r) sc[tt][r] = valid ? sc[tt][r] : kNegMax;
      }
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const float mn = fmaxf(m[r], HalfMax32(fmaxf(sc[0][r], sc[1][r])));
        alpha[r] = __builtin_amdgcn_exp2f(m[r] - mn);
        m[r] = mn;
        const float p0 = __builtin_amdgcn_exp2f(sc[0][r] - mn), p1 = __builtin_amdgcn_exp2f(sc[1][r] - mn);
        lsum[r] = __builtin_fmaf(lsum[r], alpha[r], p0 + p1);
        lp[4 * half + r][n32] = static_cast<_Float16>(p0);
        lp[4 * half + r][32 + n32] = static_cast<_Float16>(p1);
      }
      if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.0f || alpha[1] != 1.0f || alpha[2] != 1.0f || alpha[3] != 1.0f) != 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[nt][r] *= alpha[r];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      pv(tile, 0, live16);
      fetch_v(tile, 1, pgc);
      idx = nidx;
      ptile = tile;
      pace();
      if (!has_next) break;
      tile = ntile;
      pgc = pgn;
    }
    pv(ptile, 1, live16);
    leave_partial();
    __builtin_amdgcn_s_waitcnt(0);  // the slot's last copy (issued for a tile that is not coming) has landed
    __builtin_amdgcn_wave_barrier();
  }
  do {
    if (!worked) leave_empty();
    worked = false;
  } while (NextPair(a, chunk_n, &cur));
  if (a.stamps != nullptr && lane == 0) atomicMax(&a.stamps[a.n_chunks + blockIdx.x], wall_clock64());
}

// ---- the merge, with the open tile and the step's token -----------------------------------------------------------------

constexpr int kReduceDepth = 4;  // (the merge's width is its template argument: 256, 512 or 1024 threads)
constexpr int kReduceMinDims = 32;
constexpr int kTail = 17;  // keys the merge adds itself: up to 16 of the open tile, one of them the step's new token

// One workgroup per (query head, sequence, stretch of dims), as DattnReduce of decode.hip, plus the keys the split-K
// kernel leaves out: those of the sequence's newest 16-key tile, whose K is in the pools as codes and whose V is in the
// open f16 tile; in the step form the newest of them is the step's own token, which is quantized here with the append
// kernels' functions, scored from its codes as the reference's part_q would (the K append runs first there,
// loom_decoder.hpp:254-261), and written to the pools by the workgroup of the group's first query head.
template <int RT>
__global__ __launch_bounds__(RT) void Kv8Reduce(const DecodeArgs a, const Kv8Pools pools, const StepRows rows) {
  const Geom g = a.g;
  const Kv8Geom kg8{g.n_q, g.n_kv, g.n_pages, Kv8BitsK(g.format), Kv8BitsV(g.format)};
  const bool k4 = kg8.kb == 4;
  constexpr int D = kKv8Dim;
  const int G = g.group(), H = g.n_kv;
  const int hq = blockIdx.x, s = blockIdx.y, t = threadIdx.x;
  const int h = hq / G, gi = hq % G;
  const int DZ = D >> __builtin_ctz(gridDim.z), d0 = blockIdx.z * DZ;
  const size_t o = (size_t(s) * g.n_q + hq) * D + d0;
  const bool step = rows.k != nullptr;
  const int len = min(max(a.seq_len[s], 0), a.max_len);
  const int ts = TilesOf(a, s);
  __shared__ float tail_score[kTail];
  __shared__ __align__(16) float new_v[D];
  __shared__ __align__(16) float qrot[D];  // 4-bit K: the head's rotated query, H256 q / 16 rounded to f16
  if (len <= 0) {
    for (int d = t; d < DZ; d += RT) a.out[o + d] = 0.0f;
    return;
  }
  size_t p0 = 0, p1 = 0;
  if (ts > 0) {
    // (with the kv heads dealt to the waves the sequence is one pair on the line, and this head's partials lie among
    // those of all the chunks that hold a piece of the sequence)
    const int Hc = CutHeads(a);
    const long long A_ = ChunkUnits(a, static_cast<long long>(a.tprefix[a.n_seqs]) * Hc);
    const int pair = s * H + h;
    const long long first = static_cast<long long>(a.tprefix[s]) * Hc +
                            static_cast<long long>(Hc == 1 ? 0 : h) * UnitsOf(a, ts) + a.pair_cost;
    const int k0 = ChunkOf(a, A_, first), k1 = ChunkOf(a, A_, first + ts - 1);
    p0 = size_t(k0 + pair) * a.wpc, p1 = size_t(k1 + pair + 1) * a.wpc;
    if (Hc == 1 && H > 1) {
      const size_t row = size_t(h) * (a.n_chunks + a.n_seqs) + s;
      p0 = (row + k0) * a.wpc, p1 = (row + k1 + 1) * a.wpc;
    }
  }
  // The first places' (maximum, sum) entries are asked for here, before the open tile and the step's token are worked on,
  // so that their way from memory overlaps that work; they stay in registers for the sweep below.
  float2 first_ml = {kNegMax, 0.0f};
  if (p0 + t < p1) first_ml = *reinterpret_cast<const float2*>(&a.ml[((p0 + t) * G + gi) * 2]);
  if (k4) {  // the butterfly of the part kernel's prologue, over LDS (gen_decode_attn.py:655-683)
#pragma clang fp contract(off)
    if (t < D) qrot[t] = static_cast<float>(SaturateToF16(LoadSrc(a.q, (size_t(s) * g.n_q + hq) * D + t, a.q_dtype)));
    __syncthreads();
    for (int st = 1; st < D; st <<= 1) {
      if (t < D / 2) {
        const int i = (t / st) * 2 * st + t % st;
        const float lo = qrot[i], up = qrot[i + st];
        qrot[i] = lo + up, qrot[i + st] = lo - up;
      }
      __syncthreads();
    }
    if (t < D) qrot[t] = static_cast<float>(static_cast<_Float16>(qrot[t] * 0.0625f));
    __syncthreads();
  }
  const int closed = (len - 1) & ~15;           // keys the split-K kernel covered
  const int n_pool = step ? len - 1 : len;      // keys whose rows are in the pools
  const int n_tail = n_pool - closed;           // of them in the newest tile: 0 .. 16
  const int32_t* trow = a.table + int64_t(s) * a.stride;
  const int page = ClampPage(trow[min(closed / kKv8Page, a.stride - 1)], g.n_pages);
  const int page0 = ClampPage(trow[0], g.n_pages);
  // the open tile's V values of this thread's dim (the last loop below has one pass: DZ <= 256 threads), asked for now
  uint4 vo_lo = {0u, 0u, 0u, 0u}, vo_hi = vo_lo;
  if (n_tail > 0 && t < DZ) {
    const uint16_t* vo = pools.vo + kg8.vo_head(page, h) + size_t(d0 + t) * 16;
    vo_lo = *reinterpret_cast<const uint4*>(vo), vo_hi = *reinterpret_cast<const uint4*>(vo + 8);
  }
  // ---- scores of the open tile's keys: thread = (key t / 16, 16 dims of the head)
  {
    const int j = t / 16, c = t % 16;
    float part = 0.0f;
    if (j < n_tail && k4) {  // 16 dims = two dwords of one group: u * (S / 16) + (C + S), gen_decode_attn.py:806-850
      const size_t r = size_t(page) * kKv8Page + closed % kKv8Page + j;
      const uint2 w = *reinterpret_cast<const uint2*>(pools.kq + kg8.kq_row(r, h) + 2 * c);
      const uint32_t pair = pools.ks[kg8.ks_row(r, h) + c / 2];
      const float S = WidenF16(static_cast<uint16_t>(pair & 0xFFFF)), C = WidenF16(static_cast<uint16_t>(pair >> 16));
      const float d = S * 0.0625f, l0 = C + S;
      const uint32_t ww[2] = {w.x, w.y};
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int e = i % 8;
        const float u = static_cast<float>((ww[i / 8] >> (4 * (e / 2) + (e % 2 ? 16 : 0))) & 15u);
        part += (u * d + l0) * qrot[16 * c + i];
      }
    } else if (j < n_tail) {
      const size_t r = size_t(page) * kKv8Page + closed % kKv8Page + j;
      const uint4 w = *reinterpret_cast<const uint4*>(pools.kq + kg8.kq_row(r, h) + 4 * c);
      const uint32_t pair = pools.ks[kg8.ks_row(r, h) + c / 8];
      const uint32_t ww[4] = {w.x, w.y, w.z, w.w};
      const size_t qi = (size_t(s) * g.n_q + hq) * D + 16 * c;
      uint4 rq[4];  // the sixteen query values, asked for together under one branch on the type
      if (a.q_dtype == YAHKV_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) rq[i] = LoadRaw4(a.q, qi + 4 * i, YAHKV_F32);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) rq[i] = LoadRaw4(a.q, qi + 4 * i, YAHKV_F16);  // (8 bytes for bf16 as well)
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 q4 = Widen4(rq[i], a.q_dtype);
        const float qe[4] = {static_cast<float>(SaturateToF16(q4.x)), static_cast<float>(SaturateToF16(q4.y)),
                             static_cast<float>(SaturateToF16(q4.z)), static_cast<float>(SaturateToF16(q4.w))};
        // byte slots (d0, d2, d1, d3)
        part += (static_cast<float>(ww[i] & 255u) - 128.0f) * qe[0] + (static_cast<float>((ww[i] >> 16) & 255u) - 128.0f) * qe[1] +
                (static_cast<float>((ww[i] >> 8) & 255u) - 128.0f) * qe[2] + (static_cast<float>(ww[i] >> 24) - 128.0f) * qe[3];
      }
      part *= WidenF16(static_cast<uint16_t>(pair & 0xFFFF)) * 0.00390625f;
    }
    part += Dpp<kQuadSwap1>(part);
    part += Dpp<kQuadSwap2>(part);
    part += Dpp<kHalfMirror>(part);
    part += Dpp<kRowMirror>(part);
    if (c == 0 && j < n_tail) tail_score[j] = part * a.scale;
  }
  // ---- the step's token: wave 0 takes its K row, wave 1 its V row (64 lanes x 4 dims = the head)
  if (step) {
    const int wave = t / 64, lane = t % 64;
    const bool writes = gi == 0 && blockIdx.z == 0;
    const int pos = len - 1;
    const int wpage = ClampPage(trow[min(pos / kKv8Page, a.stride - 1)], g.n_pages);
    const size_t src = (size_t(s) * H + h) * D + 4 * lane;
    if (wave == 0 && k4) {
#pragma clang fp contract(off)
      const float4 x = Load4(rows.k, src, rows.dtype);
      const float4 mean = *reinterpret_cast<const float4*>(pools.km + kg8.km_head(page0, h) + 4 * lane);
      const float4 c = {TruncF16(x.x) - mean.x, TruncF16(x.y) - mean.y, TruncF16(x.z) - mean.z, TruncF16(x.w) - mean.w};
      uint32_t pair;
      float4 deq;
      uint32_t w = Kv4CodesK(c, lane, &pair, &deq);
      w |= __shfl_xor(w, 1, 64);
      if (writes) {
        const size_t r = size_t(wpage) * kKv8Page + pos % kKv8Page;
        if (lane % 2 == 0) pools.kq[kg8.kq_row(r, h) + lane / 2] = w;
        if (lane % 8 == 0) pools.ks[kg8.ks_row(r, h) + lane / 8] = pair;
      }
      const float4 q4 = *reinterpret_cast<const float4*>(&qrot[4 * lane]);
      float dot = deq.x * q4.x + deq.y * q4.y + deq.z * q4.z + deq.w * q4.w;
      dot = WaveSum(dot);
      if (lane == 0) tail_score[n_tail] = dot * a.scale;
    } else if (wave == 0) {
#pragma clang fp contract(off)
      const float4 x = Load4(rows.k, src, rows.dtype);
      const float4 mean = *reinterpret_cast<const float4*>(pools.km + kg8.km_head(page0, h) + 4 * lane);
      const float4 c = {TruncF16(x.x) - mean.x, TruncF16(x.y) - mean.y, TruncF16(x.z) - mean.z, TruncF16(x.w) - mean.w};
      float amax = fmaxf(fmaxf(fabsf(c.x), fabsf(c.y)), fmaxf(fabsf(c.z), fabsf(c.w)));
#pragma unroll
      for (int off = 16; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off, 64));
      float inv;
      uint32_t pair;
      Kv8ScaleK(amax, &inv, &pair);
      const uint32_t codes = Kv8CodesK(c, inv);
      if (writes) {
        const size_t r = size_t(wpage) * kKv8Page + pos % kKv8Page;
        pools.kq[kg8.kq_row(r, h) + lane] = codes;
        if (lane % 32 == 0) pools.ks[kg8.ks_row(r, h) + lane / 32] = pair;
      }
      const float4 q4 = Load4(a.q, (size_t(s) * g.n_q + hq) * D + 4 * lane, a.q_dtype);
      float dot = (static_cast<float>(codes & 255u) - 128.0f) * static_cast<float>(SaturateToF16(q4.x)) +
                  (static_cast<float>((codes >> 16) & 255u) - 128.0f) * static_cast<float>(SaturateToF16(q4.y)) +
                  (static_cast<float>((codes >> 8) & 255u) - 128.0f) * static_cast<float>(SaturateToF16(q4.z)) +
                  (static_cast<float>(codes >> 24) - 128.0f) * static_cast<float>(SaturateToF16(q4.w));
      dot *= WidenF16(static_cast<uint16_t>(pair & 0xFFFF)) * 0.00390625f;
      dot = WaveSum(dot);
      if (lane == 0) tail_score[n_tail] = dot * a.scale;
    } else if (wave == 1) {
      const float4 v = Load4(rows.v, src, rows.dtype);
      const float ve[4] = {v.x, v.y, v.z, v.w};
      const int key = pos % 16;
      *reinterpret_cast<float4*>(&new_v[4 * lane]) = float4{TruncF16(v.x), TruncF16(v.y), TruncF16(v.z), TruncF16(v.w)};
      if (writes) {
        uint16_t* vo = pools.vo + kg8.vo_head(wpage, h) + size_t(4 * lane) * 16;
#pragma unroll
        for (int e = 0; e < 4; ++e) vo[e * 16 + key] = F16Bits(ve[e]);
        if (key == 15) {  // the tile's 16th key: quantize it into its place (yah_dattn_vappend)
          const size_t pt = size_t(wpage) * 16 + (pos / 16) % 16;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const uint4 lo = *reinterpret_cast<const uint4*>(vo + e * 16), hi = *reinterpret_cast<const uint4*>(vo + e * 16 + 8);
            const uint32_t w[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
            float x[16];
#pragma unroll
            for (int j = 0; j < 16; ++j) x[j] = WidenF16(static_cast<uint16_t>(w[j / 2] >> (16 * (j % 2))));
            x[15] = TruncF16(ve[e]);
            uint32_t stats;
            if (kg8.vb == 4) {
              uint2 codes;
              Kv4QuantTile(x, &codes, &stats);
              *reinterpret_cast<uint2*>(pools.vq + kg8.vq_tile(h, pt) + size_t(4 * lane + e) * 2) = codes;
            } else {
              uint4 codes;
              Kv8QuantTile(x, &codes, &stats);
              *reinterpret_cast<uint4*>(pools.vq + kg8.vq_tile(h, pt) + size_t(4 * lane + e) * 4) = codes;
            }
            pools.vs[kg8.vs_tile(h, pt) + 4 * lane + e] = stats;
          }
        }
      }
    }
  }
  const int n_extra = n_tail + (step ? 1 : 0);  // 1 .. 17
  constexpr int NW = RT / 64;
  __shared__ float wgt[RT], wl[RT];
  __shared__ int slot[RT];
  __shared__ float red[NW];
  __shared__ int wave_n[NW];
  __shared__ __align__(16) float sums[RT * 4];
  __shared__ float lsums[RT / (kReduceMinDims / 4)];
  float M = first_ml.y > 0.0f ? first_ml.x : kNegMax;
  for (size_t p = p0 + t + RT; p < p1; p += RT)
    if (a.ml[(p * G + gi) * 2 + 1] > 0.0f) M = fmaxf(M, a.ml[(p * G + gi) * 2]);
  M = WaveMax(M);
  if (t % 64 == 0) red[t / 64] = M;
  __syncthreads();  // (also: the tail's scores and the new token's V row are in LDS)
  M = red[0];
  for (int w = 1; w < NW; ++w) M = fmaxf(M, red[w]);
  for (int j = 0; j < n_extra; ++j) M = fmaxf(M, tail_score[j]);
  const int lg_lanes = __builtin_ctz(static_cast<unsigned>(DZ)) - 2;
  const int lanes = 1 << lg_lanes, n_groups = RT >> lg_lanes, grp = t >> lg_lanes, dl = t & (lanes - 1);
  float L = 0.0f;
  float4 A = {0.0f, 0.0f, 0.0f, 0.0f};
  for (size_t b0 = p0; b0 < p1; b0 += RT) {
    const int nb = static_cast<int>(min(p1 - b0, size_t(RT)));
    float l = 0.0f, mm = 0.0f;
    if (b0 == p0) l = first_ml.y, mm = first_ml.x;
    else if (t < nb) l = a.ml[((b0 + t) * G + gi) * 2 + 1], mm = a.ml[((b0 + t) * G + gi) * 2];
    const unsigned long long mask = __ballot(l > 0.0f);
    __syncthreads();
    if (t % 64 == 0) wave_n[t / 64] = __popcll(mask);
    __syncthreads();
    int at = __popcll(mask & ((1ull << (t % 64)) - 1)), n = 0;
    for (int w = 0; w < NW; ++w) {
      if (w < t / 64) at += wave_n[w];
      n += wave_n[w];
    }
    if (l > 0.0f) {
      const float w = __expf(mm - M);
      wgt[at] = w, wl[at] = w * l, slot[at] = t;
    }
    __syncthreads();
    for (int j0 = grp * kReduceDepth; j0 < n; j0 += n_groups * kReduceDepth) {
      float4 v[kReduceDepth];
#pragma unroll
      for (int j = 0; j < kReduceDepth; ++j)
        v[j] = *reinterpret_cast<const float4*>(&a.acc[((b0 + slot[min(j0 + j, n - 1)]) * G + gi) * D + d0 + 4 * dl]);
#pragma unroll
      for (int j = 0; j < kReduceDepth; ++j) {
        if (j0 + j < n) {
          const float w = wgt[j0 + j];
          A.x = __builtin_fmaf(w, v[j].x, A.x), A.y = __builtin_fmaf(w, v[j].y, A.y);
          A.z = __builtin_fmaf(w, v[j].z, A.z), A.w = __builtin_fmaf(w, v[j].w, A.w);
          L += wl[j0 + j];
        }
      }
    }
  }
  *reinterpret_cast<float4*>(&sums[grp * DZ + 4 * dl]) = A;
  if (dl == 0) lsums[grp] = L;
  __syncthreads();
  for (int d = t; d < DZ; d += RT) {
    float v = 0.0f, lt = 0.0f;
    for (int q = 0; q < n_groups; ++q) v += sums[q * DZ + d], lt += lsums[q];
    // the open tile's keys, as partials of one key each: V from the open f16 tile, the step's token from its source row
    const uint32_t w[8] = {vo_lo.x, vo_lo.y, vo_lo.z, vo_lo.w, vo_hi.x, vo_hi.y, vo_hi.z, vo_hi.w};  // (d == t)
    for (int j = 0; j < n_extra; ++j) {
      const float wj = __expf(tail_score[j] - M);
      const float x = j < n_tail ? WidenF16(static_cast<uint16_t>(w[j / 2] >> (16 * (j % 2)))) : new_v[d0 + d];
      v = __builtin_fmaf(wj, x, v), lt += wj;
    }
    v /= lt;
    if (a.gate != nullptr) v *= 1.0f / (1.0f + __expf(-a.gate[o + d]));
    a.out[o + d] = v;
  }
}

int Fill(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table, int32_t stride,
         const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
         void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt, DecodeArgs* a) {
  if (const int rc = CheckKv8Pools(g, pools)) return rc;
  if (page_table == nullptr || q == nullptr || (reinterpret_cast<uintptr_t>(q) & 15)) return YAHKV_ERR_ARG;
  if (q_dtype != YAHKV_F32 && q_dtype != YAHKV_F16 && q_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if (MakeTuning(opt).one_launch) return YAHKV_ERR_ARG;
  if (const int rc = Prepare(MakeGeom(*g), stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, a)) return rc;
  a->table = page_table, a->q = q, a->q_dtype = q_dtype, a->scale = softmax_scale, a->open_tile = 1;
  if (g->n_kv_heads > 1 && kWavesPerGroup % g->n_kv_heads == 0) a->tile_mult = g->n_kv_heads;
  return YAHKV_OK;
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

static int LaunchKv8Part(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const DecodeArgs& a, hipStream_t st) {
  const dim3 grid(static_cast<unsigned>(a.n_chunks)), block(64 * kWavesPerGroup);
  const Kv8Pools p = MakeKv8Pools(*pools);
  switch (g->format) {
    case YAHKV_KV8A16: hipLaunchKernelGGL((Kv8Part<8, 8>), grid, block, 0, st, a, p); break;
    case YAHKV_KV4A16: hipLaunchKernelGGL((Kv8Part<4, 4>), grid, block, 0, st, a, p); break;
    case YAHKV_K8V4A16: hipLaunchKernelGGL((Kv8Part<8, 4>), grid, block, 0, st, a, p); break;
    default: hipLaunchKernelGGL((Kv8Part<4, 8>), grid, block, 0, st, a, p); break;
  }
  return LaunchStatus();
}

extern "C" size_t yahkv_kv8_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                                   const yahkv_decode_options* opt) {
  if (CheckKv8Geometry(g) || n_seqs <= 0 || max_seq_len <= 0) return 0;
  return MakePlan(MakeGeom(*g), n_seqs, max_seq_len, MakeTuning(opt)).bytes;
}

extern "C" int yahkv_kv8_decode_part(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                                     int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                     int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                     void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt,
                                     void* stream) {
  DecodeArgs a;
  if (const int rc = Fill(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q, q_dtype, softmax_scale,
                          workspace, workspace_bytes, opt, &a))
    return rc;
  return LaunchKv8Part(g, pools, a, static_cast<hipStream_t>(stream));
}

extern "C" int yahkv_kv8_decode_calibrate(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                                          int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                          int32_t max_seq_len, const void* q, int32_t q_dtype, void* workspace,
                                          size_t workspace_bytes, yahkv_decode_options* opt, int32_t rounds,
                                          void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto prepare = [&](DecodeArgs* a) -> int {
    return Fill(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q, q_dtype, 1.0f, workspace,
                workspace_bytes, opt, a);
  };
  auto launch = [&](const DecodeArgs& a) -> int { return LaunchKv8Part(g, pools, a, st); };
  return CalibrateXcds(prepare, launch, workspace, n_seqs, max_seq_len, opt, rounds, st);
}

extern "C" int yahkv_kv8_decode_reduce(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                                       int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                       int32_t max_seq_len, const void* k_new, const void* v_new, int32_t new_dtype,
                                       const void* q, int32_t q_dtype, float softmax_scale, const float* gate,
                                       float* out, void* workspace, size_t workspace_bytes,
                                       const yahkv_decode_options* opt, void* stream) {
  if (out == nullptr || (reinterpret_cast<uintptr_t>(out) & 15)) return YAHKV_ERR_ARG;
  if ((k_new == nullptr) != (v_new == nullptr)) return YAHKV_ERR_ARG;
  if (k_new != nullptr) {
    if ((reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new)) & 15) return YAHKV_ERR_ARG;
    if (new_dtype != YAHKV_F32 && new_dtype != YAHKV_F16 && new_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  }
  DecodeArgs a;
  if (const int rc = Fill(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q, q_dtype, softmax_scale,
                          workspace, workspace_bytes, opt, &a))
    return rc;
  a.gate = gate, a.out = out;
  int split = 1;
  while (int64_t(a.g.n_q) * a.n_seqs * split < ComputeUnits() && a.g.hd / (2 * split) >= kReduceMinDims) split *= 2;
  const int asked = MakeTuning(opt).reduce_split;
  if (asked > 0) split = std::min(asked, a.g.hd / kReduceMinDims);
  while (a.g.hd % split != 0 || (a.g.hd / split) % 4 != 0) --split;
  // A pair's places for partials are eight per chunk its tiles lie in, and with the kv heads dealt to the waves a
  // sequence's tiles lie in every chunk of its stretch: a small batch (few sequences over many chunks) has up to a
  // thousand places per pair, which a wider workgroup weighs in one sweep instead of four.
  const int64_t places = int64_t(a.n_chunks) * a.wpc / std::max(a.n_seqs, 1) + a.wpc;
  const dim3 grid(a.g.n_q, a.n_seqs, split);
  const Kv8Pools kp = MakeKv8Pools(*pools);
  const StepRows rows{k_new, v_new, new_dtype};
  if (places > 512) hipLaunchKernelGGL(Kv8Reduce<1024>, grid, dim3(1024), 0, static_cast<hipStream_t>(stream), a, kp, rows);
  else if (places > 256) hipLaunchKernelGGL(Kv8Reduce<512>, grid, dim3(512), 0, static_cast<hipStream_t>(stream), a, kp, rows);
  else hipLaunchKernelGGL(Kv8Reduce<256>, grid, dim3(256), 0, static_cast<hipStream_t>(stream), a, kp, rows);
  return LaunchStatus();
}

extern "C" int yahkv_kv8_decode_attend(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                                       int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                       int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                       const float* gate, float* out, void* workspace, size_t workspace_bytes,
                                       const yahkv_decode_options* opt, void* stream) {
  if (out == nullptr || (reinterpret_cast<uintptr_t>(out) & 15)) return YAHKV_ERR_ARG;  // before anything is launched
  if (const int rc = yahkv_kv8_decode_part(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q,
                                           q_dtype, softmax_scale, workspace, workspace_bytes, opt, stream))
    return rc;
  return yahkv_kv8_decode_reduce(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, nullptr, nullptr,
                                 0, q, q_dtype, softmax_scale, gate, out, workspace, workspace_bytes, opt, stream);
}

extern "C" int yahkv_kv8_decode_step(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                                     int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                     int32_t max_seq_len, const void* k_new, const void* v_new, int32_t new_dtype,
                                     const void* q, int32_t q_dtype, float softmax_scale, const float* gate, float* out,
                                     void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt,
                                     void* stream) {
  if (out == nullptr || (reinterpret_cast<uintptr_t>(out) & 15)) return YAHKV_ERR_ARG;
  if (k_new == nullptr || v_new == nullptr) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new)) & 15) return YAHKV_ERR_ARG;
  if (new_dtype != YAHKV_F32 && new_dtype != YAHKV_F16 && new_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if (const int rc = yahkv_kv8_decode_part(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q,
                                           q_dtype, softmax_scale, workspace, workspace_bytes, opt, stream))
    return rc;
  return yahkv_kv8_decode_reduce(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, k_new, v_new,
                                 new_dtype, q, q_dtype, softmax_scale, gate, out, workspace, workspace_bytes, opt, stream);
}
