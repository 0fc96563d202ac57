// Paged GQA decode attention over block-quantized K/V: split-K over slices of the context, then a merge.
//
// Structure follows the reference's decode attention (engine/gpu/loom/tools/gen_decode_attn.py): `part` computes one
// partial (M, l, acc) per slice of the context for the query heads of one kv head (:97-335, quantized :576-1040),
// `reduce` merges the partials: out = (sum_s e^(M_s - M) acc_s) / (sum_s e^(M_s - M) l_s) * sigmoid(gate) (:338-411).
// Keys at or past the sequence length are masked (key < pos + 1, :145,167); the "minus infinity" is the finite
// -FLT_MAX the reference uses (:357), so that no inf - inf can appear.
//
// The reference launches one workgroup per 256-key page of its single sequence. Here lengths are ragged and live on
// the device, so the work is cut stream-K style: all (sequence, kv head) pairs are laid end to end on one line of
// 64-key tiles and the line is cut into equal chunks, one per workgroup, one workgroup per CU: every CU gets the same
// number of tiles whatever the mix of lengths, in a single round. Inside a workgroup the waves take the chunk's tiles
// one by one from an LDS counter, because waves of one CU do not run at one speed (the older wave of a SIMD wins the
// issue arbitration); each wave keeps its own online softmax and leaves one partial per pair it worked on. Every
// workgroup computes its piece of the cut from the device-resident lengths itself.
// (Measured and dropped: finishing the line with short chunks or single tiles handed out dynamically, by a counter in
// global memory or by the dispatcher, to even out the XCDs, which finish up to 10 % apart. Every variant was slower:
// each change of pair costs a wave a pipeline fill, and the XCDs that finish first leave their bandwidth to the rest.)
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <mutex>
#include <vector>

#include "common.hpp"
#include "decode_cut.hpp"
#include "quant.hpp"

namespace yahkv {
namespace {


// ---- the part kernel, on the matrix cores -----------------------------------------------------------------------------
//
// A scalar-ALU version of this kernel needs 7 lane operations per q8_0 byte (one convert and one multiply-add per
// query head of the group): at 5.6 TB/s that is every VALU issue slot of the chip. So the two contractions go to MFMA,
// whose f16 rate leaves both at a few percent of peak, and the VALU only converts codes (about 1.5 operations per
// q8_0 byte, 3 per q4_0 byte):
//   scores  S[head][key] = sum_block ks[key][block] * (Q_block . codes_block)       v_mfma_f32_32x32x16_f16, one
//           32-dim block per pair of instructions (K = 16 each), so the block scale is applied to the f32 result and
//           the products themselves are exact (codes and f16 queries are exact in f16; the codes go in with the
//           constant of their f16 conversion still on, and what that adds comes off the block's sum: `lcorr`)
//   output  O[head][dim] += sum_key P[head][key] * (vs[key][block] * codes)          v_mfma_f32_16x16x32_f16; the scale
//           varies along the contraction here, so V is dequantized to f16 (one rounding, 2^-12 relative)
// The page layouts are chosen for these operand shapes. q8_0: a lane's 16-byte load is 16 dims of one key (K, [block]
// [key][32]) or 16 keys of one dim (V^T, [dim][key]). q4_0: a lane's 8-byte K load is half a block of one key (low
// nibbles dims 8 h + 0..7, high nibbles dims 16 + 8 h + 0..7, [block][key][16]); its 16-byte V load is 16 keys of the
// byte row that holds dims j and j + 16 of a block ([block][16][key]), which feeds two 16-dim output tiles.

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

// Eight nibbles of two dwords as eight f16 holding (nibble - 8), exact. Low nibbles: 0x6400 | n is 1024 + n. High
// nibbles stay in place: 0x6400 | (n << 4) is 1024 + 16 n, and one fused multiply-add takes it to n - 8.
__device__ __forceinline__ h8v NibblesLo8(uint32_t w0, uint32_t w1) {
  const h2v off = {static_cast<_Float16>(-1032.0f), static_cast<_Float16>(-1032.0f)};
  const uint32_t x0 = w0 & 0x0F0F0F0Fu, x1 = w1 & 0x0F0F0F0Fu;
  const h2v a = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u)) + off;
  const h2v b = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u)) + off;
  const h2v c = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u)) + off;
  const h2v d = __builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u)) + off;
  return h8v{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}
__device__ __forceinline__ h8v NibblesHi8(uint32_t w0, uint32_t w1) {
  const h2v mul = {static_cast<_Float16>(0.0625f), static_cast<_Float16>(0.0625f)};
  const h2v off = {static_cast<_Float16>(-72.0f), static_cast<_Float16>(-72.0f)};
  const uint32_t x0 = w0 & 0xF0F0F0F0u, x1 = w1 & 0xF0F0F0F0u;
  const h2v a = __builtin_elementwise_fma(__builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u)), mul, off);
  const h2v b = __builtin_elementwise_fma(__builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u)), mul, off);
  const h2v c = __builtin_elementwise_fma(__builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u)), mul, off);
  const h2v d = __builtin_elementwise_fma(__builtin_bit_cast(h2v, __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u)), mul, off);
  return h8v{a[0], a[1], b[0], b[1], c[0], c[1], d[0], d[1]};
}

// The same without the subtraction, for the first product: 1024 + 128 + code (q8_0), 1024 + nibble (low nibbles),
// 1024 + 16 * nibble (high nibbles, in place). What the constants add to a score depends on the queries alone and is
// taken off the block's sum afterwards (see `lcorr` in the kernel).
__device__ __forceinline__ h8v RawCodes8(uint32_t w0, uint32_t w1) {
  const uint32_t x0 = w0 ^ 0x80808080u, x1 = w1 ^ 0x80808080u;
  const uint4 r = {__builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u),
                   __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u)};
  return __builtin_bit_cast(h8v, r);
}
template <uint32_t MASK>
__device__ __forceinline__ h8v RawNibbles8(uint32_t w0, uint32_t w1) {
  const uint32_t x0 = w0 & MASK, x1 = w1 & MASK;
  const uint4 r = {__builtin_amdgcn_perm(0x64646464u, x0, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, x0, 0x04030402u),
                   __builtin_amdgcn_perm(0x64646464u, x1, 0x04010400u), __builtin_amdgcn_perm(0x64646464u, x1, 0x04030402u)};
  return __builtin_bit_cast(h8v, r);
}



// A workgroup announces that its partials of a pair are written; true for the one that is last of `n`, which then owns
// the merge. The ticket is a plain count that starts at zero: yahkv_decode_workspace_init zeroes the tickets once, and
// the last arrival of every launch puts the zero back, so launch after launch and graph replay after graph replay find
// it clean. (Relaxed atomics at device scope: the partials themselves travel by device-scope buffer accesses, written
// through and waited for before the arrival, read past the L2 after it; a release / acquire pair here would write back
// and invalidate whole L2s instead, which cost the kernel 12 % when measured.)
__device__ __forceinline__ int Arrive(unsigned long long* ticket, uint32_t n) {
  const unsigned long long old = __hip_atomic_fetch_add(ticket, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (static_cast<uint32_t>(old) + 1 != n) return 0;
  __hip_atomic_store(ticket, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // everybody has arrived
  return 1;
}

// One workgroup of eight waves per chunk, one workgroup per CU (two waves per SIMD). The waves share nothing but the
// LDS counter that hands out the chunk's tiles; after the first barrier no wave waits for another. A wave takes tiles
// in increasing order, so it meets the chunk's (sequence, kv head) pairs in order; for each pair it worked on it keeps
// an online softmax over its tiles and leaves one partial, for a pair it got no tile of it leaves l = 0.
//
// Registers hold half a tile of K (32 keys) and half a tile of V (half the dims) at a time, which keeps the kernel
// within 256 registers; the four requests of a tile are rotated against the four arithmetic phases so that every
// request has arithmetic between its issue and the first use of its data:
//   scores(keys 0-31)              | K keys 32-63 requested after it
//   P.V(dims D/2.., previous tile) | V dims 0..D/2 of this tile requested
//   scores(keys 32-63)             | K keys 0-31 of the wave's next tile requested after it
//   softmax, P.V(dims 0..D/2)      | V dims D/2.. of this tile requested
// K loads into the registers the scores have just freed. For q8_0, V loads into an LDS slot of the wave instead and
// is copied to registers right before its product, so its request goes out before that product (fetch_v / take_v);
// for q4_0, V loads into registers after the product. Page numbers come through scalar loads (they are the same
// for the whole wave).
// FUSED: the one-launch form, whose merge follows the split-K work in the same kernel. It is a template argument and
// not a field of the arguments because the merge's registers would otherwise be the plain kernel's too (spills).
// MODE 2: two dispatches as MODE 0, but what the waves have of the chunk's LAST pair meets in LDS and leaves as one
// partial instead of eight (the in-LDS merge of the one-launch form, without its tickets). For a small batch, where a
// chunk is a few tiles of a single pair, that is an eighth of the partials to write here and to read in the merge.
template <int FMT, int D, int PT, int MODE>
__global__ __launch_bounds__(64 * kWavesPerGroup) __attribute__((amdgpu_waves_per_eu(2, 2)))
void DattnPart(const DecodeArgs a) {
  constexpr bool FUSED = MODE == 1, HOLD = MODE != 0;
  constexpr int NB = D / 32, NT = D / 16, PPT = kTile / PT;
  constexpr bool Q8 = FMT == 8;
  constexpr int KW = Q8 ? 4 : 2;             // dwords of K codes per lane and block
  constexpr int NVB = Q8 ? NT / 2 : NB / 2;  // 16-byte V loads per lane and half of the dims
  constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
  const int n32 = lane % 32, half = lane / 32;  // score layout: lane = key (mod 32), registers = heads 4 * half + r
  const int n16 = lane % 16, kg = lane / 16;    // P.V layout: lane = dim (mod 16), 16 keys per lane group

  // Query A-operands [block][K half of the block's instruction pair][lane half][head row]: 8 f16 each. Row m of the
  // 32-row A matrix is head m; only rows 0-7 exist here and lanes of rows 8-31 re-read them (their output rows are
  // never looked at). Entry (b, sub, hf, row) holds the dims of the 8 codes a key lane of that half feeds to
  // instruction `sub`: 32 b + 16 hf + 8 sub + 0..7 for q8_0 (bytes 8 sub .. of its 16), 32 b + 16 sub + 8 hf + 0..7
  // for q4_0 (low nibbles, then high nibbles, of its 8 bytes).
  // The first product runs on codes with their f16 constant still on (1152 + code for q8_0; 1024 + n for low
  // nibbles; 1024 + 16 n for high nibbles, whose queries are stored divided by 16): per block and head that adds
  // (sum of the queries of the block's dims) x 1152 for q8_0, x 1032 (low) and x 72 (high) for q4_0, the -8 of
  // the nibbles included. `lcorr` holds that sum per (block, head); it comes off the block's product before the
  // block scale goes on. The products stay exact in f32 (11 x 11 bits), and the sums of 32 of them carry an error of
  // 2^-24 of 1152 x sum |q|, which is 1e-5 of a typical score.
  __shared__ __align__(16) _Float16 lq_all[kWavesPerGroup][NB][2][2][8][8];
  __shared__ __align__(16) float lcorr_all[kWavesPerGroup][NB][8];
  __shared__ __align__(16) _Float16 lp_all[kWavesPerGroup][kMaxGroup][kTile];
  __shared__ __align__(16) _Float16 lvs_all[kWavesPerGroup][NB][kTile];
  // half a tile of V codes on its way in (q8_0); at the kernel's end, either format: the waves' sums of a merge
  __shared__ __align__(16) uint8_t lvq_all[kWavesPerGroup][FMT == 8 ? NVB * 1024 : sizeof(float) * kMaxGroup * D];
  __shared__ int next_tile;
  __shared__ int progress[kWavesPerGroup];  // tiles each wave is through with (fixed pattern only)
  __shared__ int wave_sum[kWavesPerGroup][2];
  __shared__ int4 chunk_rec;
  __shared__ long long chunk_tiles[4];  // [2], [3]: for the merge, see ChunkRecord
  __shared__ int merge_flag;
  __shared__ float merge_m[kMaxGroup], merge_l[kWavesPerGroup][kMaxGroup], merge_w[kWavesPerGroup][kMaxGroup];
  auto& lq = lq_all[wave];
  auto& lcorr = lcorr_all[wave];
  auto& lp = lp_all[wave];
  auto& lvs = lvs_all[wave];
  auto& lvq = lvq_all[wave];

  if (a.stamps != nullptr && threadIdx.x == 0) a.stamps[blockIdx.x] = wall_clock64();
  bool any_empty = false;
  const int4 rec_v = a.n_seqs <= 64 ? ChunkRecordWave(a, blockIdx.x, wave, lane, &chunk_rec, chunk_tiles, &any_empty)
                                    : ChunkRecord<64 * kWavesPerGroup>(a, blockIdx.x, wave_sum, &chunk_rec, chunk_tiles, &any_empty);
  // (the record is the same in every lane: scalar registers for it and for everything derived from it)
  const int4 rec = {__builtin_amdgcn_readfirstlane(rec_v.x), __builtin_amdgcn_readfirstlane(rec_v.y),
                    __builtin_amdgcn_readfirstlane(rec_v.z), __builtin_amdgcn_readfirstlane(rec_v.w)};
  // One launch for part and merge: sequences without keys have no pair on the line and nobody merges them, so the
  // first workgroup writes their rows of zeros (its threads have just looked at a slice of the lengths each).
  if (FUSED && blockIdx.x == 0 && any_empty) {
    constexpr int NTH = 64 * kWavesPerGroup;
    const int per = (a.n_seqs + NTH - 1) / NTH;
    const int s0 = min(static_cast<int>(threadIdx.x) * per, a.n_seqs), s1 = min(s0 + per, a.n_seqs);
    for (int s = s0; s < s1; ++s)
      if (TilesOf(a, s) == 0) {
        float4* row = reinterpret_cast<float4*>(a.out + size_t(s) * g.n_q * D);
        for (int i = 0; i < g.n_q * D / 4; ++i) row[i] = float4{0.0f, 0.0f, 0.0f, 0.0f};
      }
  }
  if (rec.x < 0) return;
  const int chunk_n = rec.w;
  // (a chunk of at most one tile per wave needs no hand-out: wave w takes tile w, and the counter's barrier is saved)
  // (cut by (sequence, tile), DecodeArgs::tile_mult: item j of a sequence is tile j / H of kv head j % H, a wave of
  // the fixed pattern keeps its head, and neighbouring waves read the heads of the same tokens side by side)
  const int lg_mult = MODE == 0 && a.tile_mult > 1 ? __builtin_ctz(static_cast<unsigned>(a.tile_mult)) : 0;
  const bool fixed_pattern = a.deterministic || chunk_n <= kWavesPerGroup || lg_mult > 0;
  int head = 0;  // the kv head of the wave's current items
  if (!fixed_pattern) {
    if (threadIdx.x == 0) next_tile = 0;
    __syncthreads();
  }
  int my_next = wave;
  // With a fixed pattern nothing evens the waves out by itself: the two waves of a SIMD do not run equally fast (the
  // older one wins the issue arbitration), the faster one runs out of tiles and leaves the SIMD to a lone wave. Each
  // wave therefore tells its SIMD's other wave (wave ^ 4) how far it is, and whoever is behind raises its priority:
  // which wave works on which tile stays fixed, and with it the bits of the result.
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
  auto take = [&]() -> int {  // the next tile of the chunk nobody has taken yet (>= chunk_n: none left)
    if (fixed_pattern) {      // wave w takes tiles w, w + 8, ...: the same sums in the same order on every run
      const int v = my_next;
      my_next += kWavesPerGroup;
      return v;
    }
    int v = 0;
    if (lane == 0) v = __hip_atomic_fetch_add(&next_tile, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    return __builtin_amdgcn_readfirstlane(v);
  };

  uint32_t kb[NB][KW];  // [block]: 16 codes of this lane's key (one 32-key half of the tile at a time)
  uint4 ksc;            // that key's NB block scales (f16)
  uint4 vb[NVB];        // 16 keys of this lane's dim, or pair of dims (one half of the dims at a time)
  uint4 vsr;         // staging of the tile's V scales: 8 keys of one block per lane
  float m[4], lsum[4], sc[2][4];
  f4v o[NT];
  const float qk_scale = a.scale * kLog2e;  // softmax in base 2
  // P rows read back as A-matrix rows: rows 0-3 are heads 0-3, rows 8-11 heads 4-7, so that a lane's output rows are
  // the heads whose running maximum it already holds (lanes 0-15: heads 0-3, lanes 32-47: heads 4-7).
  const int prow = n16 < 4 ? n16 : (n16 >= 8 && n16 < 12 ? n16 - 4 : 0);

  PairCursor cur = FirstPair(a, rec);
  const int32_t* row = nullptr;
  // The page table is read through the constant address space: nothing writes it while the kernel runs, and only
  // then does the compiler use scalar loads, which the vector memory counter does not see. As ordinary global loads
  // they would sit behind the K and V loads already in flight and drain that queue once per tile.
  typedef const int32_t __attribute__((address_space(4))) * ConstRow;
  auto load_pages = [&](int tile, int (&pg)[PPT]) {
    const ConstRow crow = (ConstRow)(reinterpret_cast<uintptr_t>(row));
#pragma unroll
    for (int j = 0; j < PPT; ++j) pg[j] = ClampPage(crow[min(tile * PPT + j, a.stride - 1)], g.n_pages);
  };
  auto page_head = [&](const int (&pg)[PPT], int tok_in_tile) -> size_t {  // (page, kv head) index of a key of the tile
    int p = pg[0];
#pragma unroll
    for (int j = 1; j < PPT; ++j) p = tok_in_tile / PT == j ? pg[j] : p;
    return size_t(p) * H + head;
  };
  // Addresses are a base per (page, kv head), which is the same for the whole wave when a tile is one page, plus a
  // 32-bit offset per lane: the form the scalar-base addressing mode of the global loads takes.
  constexpr uint32_t KB = Q8 ? 32 : 16;  // bytes of K codes per key and block
  // `live` false: a load whose result nobody uses (it keeps the count of loads in flight the same on every path, see the
  // loop): every lane then reads the start of its piece, a few lines for the whole wave instead of the piece itself.
  auto load_k = [&](int tt, const int (&pg)[PPT], bool live = true) {
    const int tk = 32 * tt + n32;
    const size_t ph = page_head(pg, tk);
    const uint32_t t = live ? tk % PT : 0u;
    const uint8_t* kp = a.pools.kq + ph * (NB * PT * KB);
    const uint32_t off = live ? t * KB + (KB / 2) * half : 0u;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      if constexpr (Q8) {
        const uint4 v = StreamLoad(reinterpret_cast<const uint4*>(kp + (b * PT * KB + off)));
        kb[b][0] = v.x, kb[b][1] = v.y, kb[b][2] = v.z, kb[b][3] = v.w;
      } else {
        const uint2 v = StreamLoad(reinterpret_cast<const uint2*>(kp + (b * PT * KB + off)));
        kb[b][0] = v.x, kb[b][1] = v.y;
      }
    }
    const uint8_t* sp = reinterpret_cast<const uint8_t*>(a.pools.ks) + ph * (PT * NB * 2) + t * (NB * 2);
    if (NB == 8) {
      ksc = StreamLoad(reinterpret_cast<const uint4*>(sp));
    } else {
      const uint2 v = StreamLoad(reinterpret_cast<const uint2*>(sp));
      ksc = uint4{v.x, v.y, 0u, 0u};
    }
  };
  // V codes do not go to registers directly: the loads write this wave's LDS slot (16 bytes per lane and load, in
  // lane order), and the registers are filled from there right before the product that uses them. The slot is free
  // again as soon as it has been read, so the next half of V is requested before that product starts and stays in
  // flight through the arithmetic; a register is only free after its last use. (LDS has room for one such slot per
  // wave, so K stays in registers.) When a tile is one page the loads go through a buffer resource of the (page, kv
  // head) region: for that form the compiler keeps exact counts of the loads in flight, whereas with the flat form
  // (pages smaller than a tile: the lanes read different pages) it waits for all of them before any loaded register
  // is used.
  // q4_0 keeps the plain register loads: that kernel is bound by instruction issue, and the detour costs it more
  // instructions than the earlier request saves.
  constexpr bool kLdsV = Q8;
  auto fetch_v = [&](int hf, const int (&pg)[PPT], bool live = true) {
    const uint32_t off = live ? n16 * PT + (16 * kg) % PT : 0u;
    if constexpr (!kLdsV) {
      const size_t ph = page_head(pg, 16 * kg);
      const uint8_t* vp = a.pools.vq + ph * (Q8 ? D * PT : NB * 16 * PT);
#pragma unroll
      for (int j = 0; j < NVB; ++j) vb[j] = StreamLoad(reinterpret_cast<const uint4*>(vp + (16 * (hf * NVB + j) * PT + off)));
    } else if constexpr (PPT == 1) {
      const size_t ph = size_t(pg[0]) * H + head;
      const auto rv = __builtin_amdgcn_make_buffer_rsrc(
          const_cast<uint8_t*>(a.pools.vq) + ph * (Q8 ? D * PT : NB * 16 * PT), 0, 0x7fffffff, 0x00020000);
#pragma unroll
      for (int j = 0; j < NVB; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rv, (__attribute__((address_space(3))) void*)(&lvq[j * 1024]), 16, off,
                                                 16 * (hf * NVB + j) * PT, 0, kStreamed);
    } else {
      const size_t ph = page_head(pg, 16 * kg);
      const uint8_t* vp = a.pools.vq + ph * (Q8 ? D * PT : NB * 16 * PT);
#pragma unroll
      for (int j = 0; j < NVB; ++j)
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)(vp + (16 * (hf * NVB + j) * PT + off)),
            (__attribute__((address_space(3))) void*)(&lvq[j * 1024]), 16, 0, kStreamed);
    }
    if (hf == 0) {  // with the first half come the tile's V scales: lane = (block, 8 keys)
      const int b = lane / 8, chunk = lane % 8;
      if (b < NB) {
        const size_t ps = page_head(pg, 8 * chunk);
        const uint32_t soff = live ? (b * PT + (8 * chunk) % PT) * 2 : 0u;
        vsr = StreamLoad(reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(a.pools.vs) + ps * (NB * PT * 2) + soff));
      }
    }
  };
  auto take_v = [&]() {
    if constexpr (!kLdsV) return;
#pragma unroll
    for (int j = 0; j < NVB; ++j) vb[j] = *reinterpret_cast<const uint4*>(&lvq[j * 1024 + lane * 16]);
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the slot has been read before the next fetch is issued
  };
  // the 8 codes of block b this lane feeds to instruction `sub` of the block's pair
  auto kcodes = [&](int b, int sub) -> h8v {
    if constexpr (Q8) return RawCodes8(kb[b][2 * sub], kb[b][2 * sub + 1]);
    return sub == 0 ? RawNibbles8<0x0F0F0F0Fu>(kb[b][0], kb[b][1]) : RawNibbles8<0xF0F0F0F0u>(kb[b][0], kb[b][1]);
  };
  // scores of the 32 keys in kb against all heads: two blocks (two accumulator chains) at a time
  auto scores = [&](int tt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) sc[tt][r] = 0.0f;
#pragma unroll
    for (int b = 0; b < NB; b += 2) {
      const h8v qa0 = *reinterpret_cast<const h8v*>(&lq[b][0][half][n32 % 8][0]);
      const h8v qa1 = *reinterpret_cast<const h8v*>(&lq[b][1][half][n32 % 8][0]);
      const h8v qb0 = *reinterpret_cast<const h8v*>(&lq[b + 1][0][half][n32 % 8][0]);
      const h8v qb1 = *reinterpret_cast<const h8v*>(&lq[b + 1][1][half][n32 % 8][0]);
      const float4 k0 = *reinterpret_cast<const float4*>(&lcorr[b][4 * half]);
      const float4 k1 = *reinterpret_cast<const float4*>(&lcorr[b + 1][4 * half]);
      const float kc0[4] = {k0.x, k0.y, k0.z, k0.w}, kc1[4] = {k1.x, k1.y, k1.z, k1.w};
      f16v c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0;
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa0, kcodes(b, 0), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb0, kcodes(b + 1, 0), c1, 0, 0, 0);
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa1, kcodes(b, 1), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb1, kcodes(b + 1, 1), c1, 0, 0, 0);
      const uint32_t w = b < 2 ? ksc.x : b < 4 ? ksc.y : b < 6 ? ksc.z : ksc.w;  // scales of blocks b, b + 1
      const float d0 = WidenF16(static_cast<uint16_t>(w & 0xFFFF)) * qk_scale;
      const float d1 = WidenF16(static_cast<uint16_t>(w >> 16)) * qk_scale;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        sc[tt][r] = __builtin_fmaf(c1[r] - kc1[r], d1, __builtin_fmaf(c0[r] - kc0[r], d0, sc[tt][r]));
      // The empty asm pins the scaled sums here, so the 32x32 accumulators die before the next pair of blocks starts
      // (otherwise every pair's accumulators stay live to the end and the kernel spills).
      asm volatile("" : "+v"(sc[tt][0]), "+v"(sc[tt][1]), "+v"(sc[tt][2]), "+v"(sc[tt][3]));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // P.V for one half of the dims, from vb, lp and lvs
  auto pv = [&](int hf) {
    const h8v pa0 = *reinterpret_cast<const h8v*>(&lp[prow][16 * kg]);
    const h8v pa1 = *reinterpret_cast<const h8v*>(&lp[prow][16 * kg + 8]);
#pragma unroll
    for (int bb = 0; bb < NB / 2; ++bb) {
      const int b = hf * (NB / 2) + bb;
      const h8v s0 = *reinterpret_cast<const h8v*>(&lvs[b][16 * kg]);
      const h8v s1 = *reinterpret_cast<const h8v*>(&lvs[b][16 * kg + 8]);
#pragma unroll
      for (int j = 0; j < 2; ++j) {  // output tile 2 b + j: dims 32 b + 16 j + 0..15
        const uint4 w = vb[Q8 ? 2 * bb + j : bb];
        const int nt = 2 * b + j;
        h8v v0, v1;
        if constexpr (Q8) {
          v0 = Codes8(w.x, w.y) * s0, v1 = Codes8(w.z, w.w) * s1;
        } else if (j == 0) {
          v0 = NibblesLo8(w.x, w.y) * s0, v1 = NibblesLo8(w.z, w.w) * s1;
        } else {
          v0 = NibblesHi8(w.x, w.y) * s0, v1 = NibblesHi8(w.z, w.w) * s1;
        }
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa0, v0, o[nt], 0, 0, 0);
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa1, v1, o[nt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // l = 0 for a pair this wave got no tile of (the reduce then skips it)
  // partial of (this chunk, this wave, the current sequence, kv head h); cut by tile, every head has a row of places
  auto part_of = [&](int h) -> size_t {
    if (lg_mult > 0) return ((size_t(h) * (a.n_chunks + a.n_seqs) + blockIdx.x + cur.s) * a.wpc + wave) * G;
    return PartialIndex(a, blockIdx.x, wave, cur) * G;
  };
  auto empty_at = [&](int h) {
    if (lane < G) StoreDevice2(DeviceBuffer(a.ml + part_of(h) * 2), lane * 8, kNegMax, 0.0f);
  };
  auto leave_empty = [&]() {
    if (lg_mult == 0) return empty_at(cur.h);
    for (int h = 0; h < H; ++h) empty_at(h);
  };
  // the pair's partial, straight from registers (natural-log units, as the reduce expects)
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
  bool worked = false;  // this wave has worked on the pair `cur`
  bool held = false;    // ... and still holds its partial of it in registers: the chunk's last pair, one-launch form
  while (true) {
    // ---- move to the pair of tile idx; pairs passed without a tile get an empty partial
    bool more = idx < chunk_n;
    while (more && idx >= cur.base + cur.n) {
      if (!worked) leave_empty();
      worked = false;
      more = NextPair(a, chunk_n, &cur);
    }
    if (!more) break;
    // ---- first tile of this wave in the pair: query rows, empty state, first loads
    constexpr int QE = NB * 32 / 64;  // lq entries per lane
    h8v qreg[QE];
    const int item = cur.first + (idx - cur.base);
    head = lg_mult > 0 ? item & (a.tile_mult - 1) : cur.h;
#pragma unroll
    for (int e = 0; e < QE; ++e) {
      const int i = lane + 64 * e, b = i / 32, sub = (i / 16) % 2, hf = (i / 8) % 2, rw = i % 8;
      qreg[e] = h8v{0, 0, 0, 0, 0, 0, 0, 0};
      if (rw < G)
        qreg[e] = LoadQ8(a.q, (size_t(cur.s) * g.n_q + size_t(head) * G + rw) * D + b * 32 +
                                   (Q8 ? 16 * hf + 8 * sub : 16 * sub + 8 * hf), a.q_dtype);
    }
    row = a.table + int64_t(cur.s) * a.stride;
    int tile = item >> lg_mult;
    int pgc[PPT], pgn[PPT];
    load_pages(tile, pgc);
    load_k(0, pgc);
    fetch_v(1, pgc, false);  // not used (the first pass has no previous tile): it keeps the count of loads in flight at
                             // the head of the loop the same as on the way round, see below
#pragma unroll
    for (int e = 0; e < QE; ++e) {
      const int i = lane + 64 * e, sub = (i / 16) % 2;
      // what the codes' constants add to the block's product for head i % 8: the four entries of a (block, head)
      // lie in lanes 8 apart
      float t = 0.0f;
#pragma unroll
      for (int k = 0; k < 8; ++k) t += static_cast<float>(qreg[e][k]);
      t *= Q8 ? 1152.0f : (sub == 0 ? 1032.0f : 72.0f);
      t += __shfl_xor(t, 8, 64);
      t += __shfl_xor(t, 16, 64);
      if (lane % 32 < 8) lcorr[i / 32][i % 8] = t;
      if constexpr (!Q8) {
        if (sub == 1) qreg[e] *= static_cast<_Float16>(0.0625f);  // high nibbles come as 16 n
      }
      *reinterpret_cast<h8v*>(&lq[i / 32][sub][(i / 8) % 2][i % 8][0]) = qreg[e];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) m[r] = kNegMax, lsum[r] = 0.0f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) o[nt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    worked = true;
    bool first = true;
    // ---- this wave's tiles of the pair
    while (true) {
      const int nidx = take();
      const bool has_next = nidx < cur.base + cur.n;  // the wave's next tile is in the same pair
      const int ntile = (cur.first + (nidx - cur.base)) >> lg_mult;
      // Every pass issues the same loads whether or not the wave has a next tile in this pair (without one it
      // reads the first half of this tile's K again and drops it): the compiler counts outstanding loads along
      // every path into a wait and takes the smallest, so a load issued on one path only turns the waits after the
      // join into waits for everything.
      load_pages(has_next ? ntile : tile, pgn);
      scores(0);
      load_k(1, pgc);
      // second half of the previous tile's P.V (lp and lvs still hold that tile), and the request for this tile's
      // first half of V: before the product when V comes through LDS, after it when the registers are the buffer
      take_v();
      if constexpr (kLdsV) fetch_v(0, pgc);
      if (!first) pv(1);
      if constexpr (!kLdsV) fetch_v(0, pgc);
      first = false;
      scores(1);
      load_k(0, pgn, has_next);
      // ---- online softmax (base 2); keys at or past len are masked by select, so stale scales cannot leak
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
        lsum[r] = __builtin_fmaf(lsum[r], alpha[r], p0 + p1);  // per lane; summed over the lanes at the end
        lp[4 * half + r][n32] = static_cast<_Float16>(p0);
        lp[4 * half + r][32 + n32] = static_cast<_Float16>(p1);
      }
      {  // V scales of the tile to LDS; scales of keys at or past len become 0, which makes their V rows 0
        const int b = lane / 8, chunk = lane % 8;
        if (b < NB) {
          uint32_t w[4] = {vsr.x, vsr.y, vsr.z, vsr.w};
          const int k0 = tile * kTile + 8 * chunk;
          if (k0 + 8 > cur.len) {
#pragma unroll
            for (int j = 0; j < 8; ++j)
              if (k0 + j >= cur.len) w[j / 2] &= j % 2 ? 0x0000FFFFu : 0xFFFF0000u;
          }
          *reinterpret_cast<uint4*>(&lvs[b][8 * chunk]) = uint4{w[0], w[1], w[2], w[3]};
        }
      }
      // once a pair's maximum has settled (a few tiles into a long sequence) every factor is exactly 1
      if (__builtin_amdgcn_ballot_w64(alpha[0] != 1.0f || alpha[1] != 1.0f || alpha[2] != 1.0f || alpha[3] != 1.0f) != 0) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[nt][r] *= alpha[r];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      take_v();  // this tile's first half of V
      if constexpr (kLdsV) fetch_v(1, pgc);
      pv(0);
      if constexpr (!kLdsV) fetch_v(1, pgc);
      idx = nidx;
      pace();
      if (!has_next) break;
      tile = ntile;
#pragma unroll
      for (int j = 0; j < PPT; ++j) pgc[j] = pgn[j];
    }
    take_v();
    pv(1);
    // One launch for part and merge: what a wave has of the chunk's last pair stays in its registers, and the waves'
    // shares of that pair meet in LDS below instead of travelling through memory one by one.
    if (HOLD && cur.base + cur.n >= chunk_n) {
      held = true;
      break;
    }
    leave_partial();
    __builtin_amdgcn_wave_barrier();  // lq, lp and lvs are rewritten for the next pair
  }
  // pairs of the chunk after this wave's last tile (of the last pair, a wave that holds nothing says so in LDS below)
  if (!held) {
    do {
      if (!worked && !(HOLD && cur.base + cur.n >= chunk_n)) leave_empty();
      worked = false;
    } while (NextPair(a, chunk_n, &cur));
  }
  if (a.stamps != nullptr && lane == 0) atomicMax(&a.stamps[a.n_chunks + blockIdx.x], wall_clock64());
  if (!HOLD) return;

  // ---- the merge, in the same launch (gen_decode_attn.py:338-411 is the reference's separate dispatch). A pair's
  // partials come from the workgroups of every chunk its tiles lie in; each of them, when all its waves are done,
  // announces itself on the pair's ticket, and the one that finds all the others already there merges the pair. Nobody
  // waits for anybody. LDS: the V slots, which nobody needs any more, hold the waves' sums.
  static_assert(sizeof(lvq_all) >= sizeof(float) * kWavesPerGroup * kMaxGroup * D, "merge sums fit the V slots");
  float* const sums = reinterpret_cast<float*>(&lvq_all[0][0]);  // [wave][head][D]
  constexpr int NTH = 64 * kWavesPerGroup;
  constexpr int VPL = D / 64;  // dims per lane
  typedef typename LoadDeviceN<VPL>::type fvv;

  // -- the chunk's last pair: the waves' shares, still in registers, are merged through LDS into one partial
  if (n32 == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) merge_w[wave][4 * half + r] = held ? m[r] : kNegMax;
  }
  __syncthreads();  // (every wave is past its last tile: the V slots are free)
  {
    float f[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float M = kNegMax;
#pragma unroll
      for (int w = 0; w < kWavesPerGroup; ++w) M = fmaxf(M, merge_w[w][4 * half + r]);
      f[r] = held ? __builtin_amdgcn_exp2f(m[r] - M) : 0.0f;
      const float l = held ? HalfSum32(lsum[r]) * f[r] : 0.0f;
      if (n32 == 0) merge_l[wave][4 * half + r] = l;
      if (n32 == 0 && wave == 0) merge_m[4 * half + r] = M;  // (log2 units)
    }
    if (kg == 0 || kg == 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
          sums[(wave * kMaxGroup + 2 * kg + r) * D + 16 * nt + n16] = held ? o[nt][r] * f[r] : 0.0f;
    }
  }
  __syncthreads();

  int4 mrec = chunk_rec;  // (read again rather than kept in registers through the tile loop)
  mrec.w = static_cast<int>(chunk_tiles[1] - chunk_tiles[0]);
  const int merge_n = mrec.w;
  const long long units_per_chunk = chunk_tiles[3];
  // writes one row of the output from the waves' sums in LDS
  auto finish = [&](int s_, int h_) {
    for (int i = threadIdx.x; i < G * D; i += NTH) {
      const int gi = i / D, d = i % D;
      float v = 0.0f, l = 0.0f;
#pragma unroll
      for (int w = 0; w < kWavesPerGroup; ++w) v += sums[(w * kMaxGroup + gi) * D + d], l += merge_l[w][gi];
      v /= l;
      const size_t o_ = (size_t(s_) * g.n_q + size_t(h_) * G + gi) * D + d;
      if (a.gate != nullptr) v *= 1.0f / (1.0f + __expf(-a.gate[o_]));
      a.out[o_] = v;
    }
  };
  // merges the partials of a pair that lie in memory: chunks k0 .. k1, eight slots each, most of them empty (a chunk
  // that held the pair as its last leaves one slot, a wave without a tile of the pair none). Memory is a few
  // microseconds away here, so everything is asked for in as few rounds as possible: all (maximum, sum) entries at
  // once for the heads' maxima; again, 512 slots at a time, for a table of weights in LDS; then every wave asks for
  // the rows of its non-empty slots, a few slots' rows together.
  static_assert(sizeof(lq_all) >= sizeof(float) * kMergeSlots * kMaxGroup, "the weights fit the query operands' LDS");
  float* const wgt = reinterpret_cast<float*>(&lq_all[0][0][0][0][0][0]);  // [slot][head], 0 for an empty slot
  auto merge = [&](int s_, int h_, int k0, int k1) {
    const int pair = s_ * H + h_;
    const size_t slot0 = size_t(k0 + pair) * a.wpc;
    const int n_slots = (k1 - k0 + 1) * a.wpc;
    const int gi = threadIdx.x % kMaxGroup, sl = threadIdx.x / kMaxGroup;  // thread = (slot mod 64, head)
    constexpr int SPT = kMergeSlots / (NTH / kMaxGroup);                   // slots per thread and sweep: 8
    float M = kNegMax;
    for (int b0 = 0; b0 < n_slots; b0 += kMergeSlots) {
      const auto rml = DeviceBuffer(a.ml + (slot0 + b0) * G * 2);
      float2 v[SPT];
#pragma unroll
      for (int u = 0; u < SPT; ++u) {
        const int j = sl + (NTH / kMaxGroup) * u;
        v[u] = gi < G && b0 + j < n_slots ? LoadDevice2(rml, (j * G + gi) * 8) : float2{kNegMax, 0.0f};
      }
#pragma unroll
      for (int u = 0; u < SPT; ++u)
        if (v[u].y > 0.0f) M = fmaxf(M, v[u].x);
    }
    // (lanes of one head are 8 apart: three steps across the wave, then the waves through LDS)
    M = fmaxf(M, __shfl_xor(M, 8, 64)), M = fmaxf(M, __shfl_xor(M, 16, 64)), M = fmaxf(M, __shfl_xor(M, 32, 64));
    if (lane < kMaxGroup) merge_w[wave][lane] = M;
    __syncthreads();
    M = kNegMax;
#pragma unroll
    for (int w = 0; w < kWavesPerGroup; ++w) M = fmaxf(M, merge_w[w][gi]);
    fvv acc[kMaxGroup];
    float L = 0.0f;  // of head gi, this thread's slots
#pragma unroll
    for (int q_ = 0; q_ < kMaxGroup; ++q_) {
#pragma unroll
      for (int e = 0; e < VPL; ++e) acc[q_][e] = 0.0f;
    }
    for (int b0 = 0; b0 < n_slots; b0 += kMergeSlots) {
      const int nb = min(n_slots - b0, kMergeSlots);
      const auto rml = DeviceBuffer(a.ml + (slot0 + b0) * G * 2);
      float2 v[SPT];
#pragma unroll
      for (int u = 0; u < SPT; ++u) {
        const int j = sl + (NTH / kMaxGroup) * u;
        v[u] = gi < G && j < nb ? LoadDevice2(rml, (j * G + gi) * 8) : float2{kNegMax, 0.0f};
      }
#pragma unroll
      for (int u = 0; u < SPT; ++u) {
        const float w = v[u].y > 0.0f ? __expf(v[u].x - M) : 0.0f;
        L = __builtin_fmaf(w, v[u].y, L);
        wgt[(sl + (NTH / kMaxGroup) * u) * kMaxGroup + gi] = w;
      }
      __syncthreads();
      // Wave w takes slot (c, r) of chunk c when (c + r) % 8 == w: a chunk's single slot (r = 0) goes to wave c % 8,
      // and the eight slots of a chunk that left all of them go to the eight waves. One r at a time, four chunks'
      // slots together.
      for (int r = 0; r < kWavesPerGroup; ++r) {
        for (int c0 = (wave - r + kWavesPerGroup) % kWavesPerGroup; c0 * kWavesPerGroup < nb; c0 += 4 * kWavesPerGroup) {
          fvv row[4][kMaxGroup];
          float wv[4][kMaxGroup];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const int j = (c0 + kWavesPerGroup * t) * kWavesPerGroup + r;
            const bool in = j < nb;
            const auto racc = DeviceBuffer(a.acc + (slot0 + b0 + (in ? j : 0)) * G * D);
#pragma unroll
            for (int q_ = 0; q_ < kMaxGroup; ++q_) {
              wv[t][q_] = in && q_ < G ? wgt[j * kMaxGroup + q_] : 0.0f;  // the same in every lane
              if (wv[t][q_] > 0.0f) row[t][q_] = LoadDeviceN<VPL>::load(racc, (q_ * D + VPL * lane) * 4);
            }
          }
#pragma unroll
          for (int t = 0; t < 4; ++t)
#pragma unroll
            for (int q_ = 0; q_ < kMaxGroup; ++q_)
              if (wv[t][q_] > 0.0f) {
#pragma unroll
                for (int e = 0; e < VPL; ++e) acc[q_][e] = __builtin_fmaf(wv[t][q_], row[t][q_][e], acc[q_][e]);
              }
        }
      }
      __syncthreads();  // the table is free for the next 512 slots
    }
    // the sums of the threads of one head (lanes 8 apart), then of the waves
    L += __shfl_xor(L, 8, 64), L += __shfl_xor(L, 16, 64), L += __shfl_xor(L, 32, 64);
    if (lane < kMaxGroup) merge_l[wave][lane] = L;
#pragma unroll
    for (int q_ = 0; q_ < kMaxGroup; ++q_)
      if (q_ < G) *reinterpret_cast<fvv*>(&sums[(wave * kMaxGroup + q_) * D + VPL * lane]) = acc[q_];
    __syncthreads();
    finish(s_, h_);
    __syncthreads();  // the sums are free for the next pair
  };

  // announces this workgroup's partials of a pair and merges the pair if all the others are in
  auto arrive_and_merge = [&](int s_, int h_, int k0, int k1) {
    // every partial of this workgroup for the pair has reached memory before the workgroup says so
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    if (threadIdx.x == 0)
      merge_flag = k0 == k1 ? 1 : Arrive(&a.tickets[s_ * H + h_], static_cast<uint32_t>(k1 - k0 + 1));
    __syncthreads();
    const bool mine = merge_flag != 0;
    __syncthreads();  // (the flag is free again)
    if (mine) merge(s_, h_, k0, k1);
  };
  // The last pair first, while its sum is in LDS: finished here if all of it was this workgroup's, else written out
  // as this chunk's one partial of it (slot 0; the other seven slots stay empty).
  {
    MergeCursor mc = FirstMergePair(a, mrec, chunk_tiles[2]);
    while (NextMergePair(a, merge_n, &mc)) {
    }
    const int s_ = mc.c.s, h_ = mc.c.h;
    const int k0 = ChunkOf(a, units_per_chunk, mc.line0), k1 = ChunkOf(a, units_per_chunk, mc.line0 + mc.ts - 1);
    if (FUSED && k0 == k1) {
      finish(s_, h_);
      __syncthreads();
    } else {
      const size_t part = (size_t(blockIdx.x) + size_t(s_) * H + h_) * a.wpc * G;
      const auto rml = DeviceBuffer(a.ml + part * 2), racc = DeviceBuffer(a.acc + part * D);
      for (int i = threadIdx.x; i < G * D; i += NTH) {
        const int gi = i / D, d = i % D;
        float v = 0.0f;
#pragma unroll
        for (int w = 0; w < kWavesPerGroup; ++w) v += sums[(w * kMaxGroup + gi) * D + d];
        StoreDevice(racc, i * 4, v);
        if (d < a.wpc) {
          float l = 0.0f;
#pragma unroll
          for (int w = 0; w < kWavesPerGroup; ++w) l += merge_l[w][gi];
          StoreDevice2(rml, (d * G + gi) * 8, merge_m[gi] * kLn2, d == 0 ? l : 0.0f);
        }
      }
      if (!FUSED) return;  // MODE 2: the separate merge dispatch takes it from here
      arrive_and_merge(s_, h_, k0, k1);
    }
  }
  // the pairs before it ended in this chunk; their partials went to memory wave by wave
  MergeCursor mc = FirstMergePair(a, mrec, chunk_tiles[2]);
  while (mc.c.base + mc.c.n < merge_n) {
    const int s_ = mc.c.s, h_ = mc.c.h;
    const int k0 = ChunkOf(a, units_per_chunk, mc.line0), k1 = ChunkOf(a, units_per_chunk, mc.line0 + mc.ts - 1);
    arrive_and_merge(s_, h_, k0, k1);
    if (!NextMergePair(a, merge_n, &mc)) break;
  }
}

// The part kernel for a batch of about one tile per wave (one long sequence, a few short ones): q8_0, head_dim 256,
// 64-token pages, so a tile is one page. The cut of the line, the partials and what the separate merge expects are
// DattnPart's in its MODE 2 (one partial per workgroup for the chunk's last pair); what differs is how a wave goes
// through a tile. With a single tile there is nothing for the rotation above to run ahead of, and its four requests,
// half a tile of K or V each, are four trips to memory one behind the other. Here a wave asks for both halves of its
// tile's K at once, next to its query rows (which it only looks at once those requests are out), and for V into the
// registers the K codes leave. Its result for the pair goes to the wave's LDS slot (V does not pass through LDS
// here), where a second tile of the same pair joins it and where the workgroup's merge finds it, so nothing but the
// tile in hand occupies registers. Wave w takes tiles w, w + 8, ... of the chunk: the same sums in the same order on
// every run.
__global__ __launch_bounds__(64 * kWavesPerGroup) __attribute__((amdgpu_waves_per_eu(2, 2)))
void DattnPartWhole(const DecodeArgs a) {
  constexpr int D = 256, PT = kTile, NB = D / 32, NT = D / 16, NVB = NT / 2, QE = NB * 32 / 64;
  constexpr int NTH = 64 * kWavesPerGroup;
  constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / 64), lane = threadIdx.x % 64;
  const int n32 = lane % 32, half = lane / 32;  // score layout: lane = key (mod 32), registers = heads 4 * half + r
  const int n16 = lane % 16, kg = lane / 16;    // P.V layout: lane = dim (mod 16), 16 keys per lane group
  // (query operands, their constants' sums, weights and V scales: the layouts of DattnPart<8, 256, 64, .>)
  __shared__ __align__(16) _Float16 lq_all[kWavesPerGroup][NB][2][2][8][8];
  __shared__ __align__(16) float lcorr_all[kWavesPerGroup][NB][8];
  __shared__ __align__(16) _Float16 lp_all[kWavesPerGroup][kMaxGroup][kTile];
  __shared__ __align__(16) _Float16 lvs_all[kWavesPerGroup][NB][kTile];
  __shared__ __align__(16) float share_all[kWavesPerGroup][kMaxGroup][D];  // a wave's sums for its current pair
  __shared__ float share_m[kWavesPerGroup][kMaxGroup], share_l[kWavesPerGroup][kMaxGroup];  // their maxima (log2) and weights
  __shared__ int4 chunk_rec;
  __shared__ long long chunk_tiles[4];
  __shared__ int wave_sum[kWavesPerGroup][2];
  auto& lq = lq_all[wave];
  auto& lcorr = lcorr_all[wave];
  auto& lp = lp_all[wave];
  auto& lvs = lvs_all[wave];
  float* const share = &share_all[wave][0][0];

  if (a.stamps != nullptr && threadIdx.x == 0) a.stamps[blockIdx.x] = wall_clock64();
  bool any_empty = false;
  const int4 rec_v = a.n_seqs <= 64 ? ChunkRecordWave(a, blockIdx.x, wave, lane, &chunk_rec, chunk_tiles, &any_empty)
                                    : ChunkRecord<NTH>(a, blockIdx.x, wave_sum, &chunk_rec, chunk_tiles, &any_empty);
  const int4 rec = {__builtin_amdgcn_readfirstlane(rec_v.x), __builtin_amdgcn_readfirstlane(rec_v.y),
                    __builtin_amdgcn_readfirstlane(rec_v.z), __builtin_amdgcn_readfirstlane(rec_v.w)};
  if (rec.x < 0) return;
  const int chunk_n = rec.w;

  uint32_t kb[2][NB][4];  // [half of the tile][block]: 16 codes of this lane's key
  uint4 ksc[2];           // that key's NB block scales (f16)
  uint4 vb[2][NVB];       // [half of the dims]: 16 keys of this lane's dim
  uint4 vsr;              // staging of the tile's V scales: 8 keys of one block per lane
  float m[4], lsum[4], sc[2][4];
  f4v o[NT];
  const float qk_scale = a.scale * kLog2e;  // softmax in base 2
  const int prow = n16 < 4 ? n16 : (n16 >= 8 && n16 < 12 ? n16 - 4 : 0);  // P rows as A-matrix rows, see DattnPart

  PairCursor cur = FirstPair(a, rec);
  typedef const int32_t __attribute__((address_space(4))) * ConstRow;  // (scalar loads, see DattnPart)
  auto load_page = [&](int tile) -> int {
    const ConstRow crow = (ConstRow)(reinterpret_cast<uintptr_t>(a.table + int64_t(cur.s) * a.stride));
    return ClampPage(crow[min(tile, a.stride - 1)], g.n_pages);
  };
  auto load_k = [&](int tt, size_t ph) {
    const uint8_t* kp = a.pools.kq + ph * (NB * PT * 32);
    const uint32_t off = (32 * tt + n32) * 32 + 16 * half;
#pragma unroll
    for (int b = 0; b < NB; ++b) {
      const uint4 v = StreamLoad(reinterpret_cast<const uint4*>(kp + (b * PT * 32 + off)));
      kb[tt][b][0] = v.x, kb[tt][b][1] = v.y, kb[tt][b][2] = v.z, kb[tt][b][3] = v.w;
    }
    ksc[tt] = StreamLoad(reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(a.pools.ks) + ph * (PT * NB * 2) +
                                                        (32 * tt + n32) * (NB * 2)));
  };
  auto load_v = [&](int hf, size_t ph) {
    const uint8_t* vp = a.pools.vq + ph * (D * PT);
    const uint32_t off = n16 * PT + 16 * kg;
#pragma unroll
    for (int j = 0; j < NVB; ++j) vb[hf][j] = StreamLoad(reinterpret_cast<const uint4*>(vp + (16 * (hf * NVB + j) * PT + off)));
  };
  auto load_vs = [&](size_t ph) {  // lane = (block, 8 keys)
    const int b = lane / 8, chunk = lane % 8;
    vsr = StreamLoad(reinterpret_cast<const uint4*>(reinterpret_cast<const uint8_t*>(a.pools.vs) + ph * (NB * PT * 2) +
                                                    (b * PT + 8 * chunk) * 2));
  };
  // scores of the 32 keys of half tt against all heads: two blocks (two accumulator chains) at a time
  auto scores = [&](int tt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) sc[tt][r] = 0.0f;
#pragma unroll
    for (int b = 0; b < NB; b += 2) {
      const h8v qa0 = *reinterpret_cast<const h8v*>(&lq[b][0][half][n32 % 8][0]);
      const h8v qa1 = *reinterpret_cast<const h8v*>(&lq[b][1][half][n32 % 8][0]);
      const h8v qb0 = *reinterpret_cast<const h8v*>(&lq[b + 1][0][half][n32 % 8][0]);
      const h8v qb1 = *reinterpret_cast<const h8v*>(&lq[b + 1][1][half][n32 % 8][0]);
      const float4 k0 = *reinterpret_cast<const float4*>(&lcorr[b][4 * half]);
      const float4 k1 = *reinterpret_cast<const float4*>(&lcorr[b + 1][4 * half]);
      const float kc0[4] = {k0.x, k0.y, k0.z, k0.w}, kc1[4] = {k1.x, k1.y, k1.z, k1.w};
      f16v c0 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}, c1 = c0;
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa0, RawCodes8(kb[tt][b][0], kb[tt][b][1]), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb0, RawCodes8(kb[tt][b + 1][0], kb[tt][b + 1][1]), c1, 0, 0, 0);
      c0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa1, RawCodes8(kb[tt][b][2], kb[tt][b][3]), c0, 0, 0, 0);
      c1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(qb1, RawCodes8(kb[tt][b + 1][2], kb[tt][b + 1][3]), c1, 0, 0, 0);
      const uint32_t w = b < 2 ? ksc[tt].x : b < 4 ? ksc[tt].y : b < 6 ? ksc[tt].z : ksc[tt].w;  // scales of blocks b, b + 1
      const float d0 = WidenF16(static_cast<uint16_t>(w & 0xFFFF)) * qk_scale;
      const float d1 = WidenF16(static_cast<uint16_t>(w >> 16)) * qk_scale;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        sc[tt][r] = __builtin_fmaf(c1[r] - kc1[r], d1, __builtin_fmaf(c0[r] - kc0[r], d0, sc[tt][r]));
      // (the accumulators die before the next pair of blocks starts, see DattnPart)
      asm volatile("" : "+v"(sc[tt][0]), "+v"(sc[tt][1]), "+v"(sc[tt][2]), "+v"(sc[tt][3]));
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // P.V for one half of the dims, from vb, lp and lvs
  auto pv = [&](int hf) {
    const h8v pa0 = *reinterpret_cast<const h8v*>(&lp[prow][16 * kg]);
    const h8v pa1 = *reinterpret_cast<const h8v*>(&lp[prow][16 * kg + 8]);
#pragma unroll
    for (int bb = 0; bb < NB / 2; ++bb) {
      const int b = hf * (NB / 2) + bb;
      const h8v s0 = *reinterpret_cast<const h8v*>(&lvs[b][16 * kg]);
      const h8v s1 = *reinterpret_cast<const h8v*>(&lvs[b][16 * kg + 8]);
#pragma unroll
      for (int j = 0; j < 2; ++j) {  // output tile 2 b + j: dims 32 b + 16 j + 0..15
        const uint4 w = vb[hf][2 * bb + j];
        const int nt = 2 * b + j;
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa0, Codes8(w.x, w.y) * s0, o[nt], 0, 0, 0);
        o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa1, Codes8(w.z, w.w) * s1, o[nt], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  auto leave_empty = [&]() {  // l = 0 for a pair this wave got no tile of (the merge then skips it)
    if (lane < G) StoreDevice2(DeviceBuffer(a.ml + PartialIndex(a, blockIdx.x, wave, cur) * G * 2), lane * 8, kNegMax, 0.0f);
  };
  // the wave is through with pair `cur`, which ends inside the chunk: its share goes to memory as the wave's partial
  auto flush = [&]() {
    const size_t part = PartialIndex(a, blockIdx.x, wave, cur) * G;
    const auto rml = DeviceBuffer(a.ml + part * 2), racc = DeviceBuffer(a.acc + part * D);
    if (lane < G) StoreDevice2(rml, lane * 8, share_m[wave][lane] * kLn2, share_l[wave][lane]);
    for (int i = lane; i < G * D; i += 64) StoreDevice(racc, i * 4, share[i]);
    __builtin_amdgcn_wave_barrier();  // (the slot is rewritten for the next pair)
  };

  bool live = false;  // the wave has a share of pair `cur` in its slot
  for (int idx = wave;; idx += kWavesPerGroup) {
    bool more = idx < chunk_n;
    while (more && idx >= cur.base + cur.n) {  // (a pair left behind by a later tile is not the chunk's last)
      if (live) flush();
      else leave_empty();
      live = false;
      more = NextPair(a, chunk_n, &cur);
    }
    if (!more) break;
    const int tile = cur.first + (idx - cur.base);
    // ---- requests: the query rows (a second tile of the same pair finds them in LDS), then K and the V scales
    RawQ8 qraw[QE];
    if (!live) {
#pragma unroll
      for (int e = 0; e < QE; ++e) {
        const int i = lane + 64 * e, b = i / 32, sub = (i / 16) % 2, hf = (i / 8) % 2, rw = i % 8;
        qraw[e] = RawQ8{uint4{0u, 0u, 0u, 0u}, uint4{0u, 0u, 0u, 0u}};  // (zero bits are zero in every query type)
        if (rw < G)
          qraw[e] = LoadRawQ8(a.q, (size_t(cur.s) * g.n_q + size_t(cur.h) * G + rw) * D + b * 32 + 16 * hf + 8 * sub, a.q_dtype);
      }
    }
    const size_t ph = size_t(load_page(tile)) * H + cur.h;
    load_k(0, ph), load_k(1, ph), load_vs(ph);
    if (!live) {
#pragma unroll
      for (int e = 0; e < QE; ++e) {
        const int i = lane + 64 * e, sub = (i / 16) % 2;
        const h8v qv = ConvertQ8(qraw[e], a.q_dtype);
        // what the codes' constants add to the block's product for head i % 8: the four entries of a (block, head)
        // lie in lanes 8 apart
        float t = 0.0f;
#pragma unroll
        for (int k = 0; k < 8; ++k) t += static_cast<float>(qv[k]);
        t *= 1152.0f;
        t += __shfl_xor(t, 8, 64);
        t += __shfl_xor(t, 16, 64);
        if (lane % 32 < 8) lcorr[i / 32][i % 8] = t;
        *reinterpret_cast<h8v*>(&lq[i / 32][sub][(i / 8) % 2][i % 8][0]) = qv;
      }
    }
    // ---- scores; V is asked for into the registers the K codes leave
    scores(0);
    load_v(0, ph);
    scores(1);
    load_v(1, ph);
    // ---- softmax (base 2) of the tile by itself; keys at or past len are masked by select
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const bool valid = tile * kTile + 32 * tt + n32 < cur.len;
#pragma unroll
      for (int r = 0; r < 4; ++r) sc[tt][r] = valid ? sc[tt][r] : kNegMax;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      m[r] = HalfMax32(fmaxf(sc[0][r], sc[1][r]));
      const float p0 = __builtin_amdgcn_exp2f(sc[0][r] - m[r]), p1 = __builtin_amdgcn_exp2f(sc[1][r] - m[r]);
      lsum[r] = HalfSum32(p0 + p1);
      lp[4 * half + r][n32] = static_cast<_Float16>(p0);
      lp[4 * half + r][32 + n32] = static_cast<_Float16>(p1);
    }
    {  // V scales of the tile to LDS; scales of keys at or past len become 0, which makes their V rows 0
      const int b = lane / 8, chunk = lane % 8;
      uint32_t w[4] = {vsr.x, vsr.y, vsr.z, vsr.w};
      const int k0 = tile * kTile + 8 * chunk;
      if (k0 + 8 > cur.len) {
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (k0 + j >= cur.len) w[j / 2] &= j % 2 ? 0x0000FFFFu : 0xFFFF0000u;
      }
      *reinterpret_cast<uint4*>(&lvs[b][8 * chunk]) = uint4{w[0], w[1], w[2], w[3]};
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) o[nt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
    pv(0), pv(1);
    // ---- the tile's result joins the wave's share of the pair
    float fo[4], fn[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      fo[r] = 0.0f, fn[r] = 1.0f;
      if (live) {
        const float mo = share_m[wave][4 * half + r], mn = fmaxf(mo, m[r]);
        fo[r] = __builtin_amdgcn_exp2f(mo - mn), fn[r] = __builtin_amdgcn_exp2f(m[r] - mn);
        lsum[r] = __builtin_fmaf(share_l[wave][4 * half + r], fo[r], lsum[r] * fn[r]);
        m[r] = mn;
      }
    }
    __builtin_amdgcn_wave_barrier();  // (every lane has read the share's maxima and weights)
    if (n32 == 0) {
#pragma unroll
      for (int r = 0; r < 4; ++r) share_m[wave][4 * half + r] = m[r], share_l[wave][4 * half + r] = lsum[r];
    }
    if (kg == 0 || kg == 2) {  // (these lanes' output rows are heads 2 kg + r)
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
          float* const at = &share[(2 * kg + r) * D + 16 * nt + n16];
          *at = live ? __builtin_fmaf(*at, fo[r], o[nt][r] * fn[r]) : o[nt][r];
        }
    }
    live = true;
    __builtin_amdgcn_wave_barrier();  // lq, lp and lvs are rewritten for the next tile
  }
  // the pair of the wave's last tile and the pairs after it; the share of the chunk's last pair stays in the slot
  bool held = false;
  do {
    if (cur.base + cur.n >= chunk_n) held = live;
    else if (live) flush();
    else leave_empty();
    live = false;
  } while (NextPair(a, chunk_n, &cur));
  if (a.stamps != nullptr && lane == 0) atomicMax(&a.stamps[a.n_chunks + blockIdx.x], wall_clock64());

  // ---- the chunk's last pair (every wave's cursor has come to rest on it): one barrier and one sweep over the row
  // leave the workgroup's partial of it, slot 0 of its eight; the other seven stay empty
  if (!held && n32 == 0) {
#pragma unroll
    for (int r = 0; r < 4; ++r) share_m[wave][4 * half + r] = kNegMax;
  }
  __syncthreads();
  const size_t part = (size_t(blockIdx.x) + size_t(cur.s) * H + cur.h) * a.wpc * G;
  const auto rml = DeviceBuffer(a.ml + part * 2), racc = DeviceBuffer(a.acc + part * D);
  for (int i = threadIdx.x; i < G * D; i += NTH) {
    const int gi = i / D, d = i % D;
    float M = kNegMax;
#pragma unroll
    for (int w = 0; w < kWavesPerGroup; ++w) M = fmaxf(M, share_m[w][gi]);
    float v = 0.0f, l = 0.0f;
#pragma unroll
    for (int w = 0; w < kWavesPerGroup; ++w) {
      const float mw = share_m[w][gi];
      if (mw > kNegMax) {  // (the slot of a wave without a share holds anything)
        const float f = __builtin_amdgcn_exp2f(mw - M);
        v = __builtin_fmaf(share_all[w][gi][d], f, v), l = __builtin_fmaf(share_l[w][gi], f, l);
      }
    }
    StoreDevice(racc, i * 4, v);
    if (d < a.wpc) StoreDevice2(rml, (d * G + gi) * 8, M * kLn2, d == 0 ? l : 0.0f);
  }
}

// ---- reduce -------------------------------------------------------------------------------------------------------------

// One workgroup per (query head, sequence) (gen_decode_attn.py:338-411). The pair's partials are those of the waves
// of the chunks its stretch of the line overlaps. Their weights e^(M_p - M) are computed once per workgroup, by one
// thread each, and the partials that weigh something are listed in order. The threads then form groups of D / 4
// lanes (four dims a lane); each group sums every n-th listed partial, several 16-byte loads in flight and no
// branch inside, and the groups' sums meet in LDS. A single long sequence leaves hundreds of partials per pair and
// only a few workgroups here, which is why the partials are spread over the workgroup as well, and why a small batch
// is launched with several workgroups per pair (gridDim.z), each with its own stretch of the head's dims: what bounds
// such a launch is the number of partial rows in flight.
//
// The step form (rows given): the sequence's newest token is not in the pools yet. The first wave quantizes its K
// row of this kv head exactly as the append kernel does (quant.hpp), takes the score of the dequantized row against
// this workgroup's query head, and the second wave does the same for the V row and leaves the dequantized values in
// LDS; the token then enters the sums like one more partial (maximum = its score, sum = 1, accumulator = its V row).
// The workgroup of the group's first query head (and first stretch of dims) also writes the codes and scales to the
// token's slot, so after the launch the pools hold what yahkv_append would have written.
__device__ __forceinline__ void StepToken(const DecodeArgs& a, const StepRows& rows, int s, int h, int hq, int wave, int lane, bool writes,
                                          float* score, float* vrow) {
  const Geom& g = a.g;
  const int D = g.hd, d0 = 4 * lane;
  const bool has = d0 < D, is_v = wave == 1;
  // everything this wave reads is asked for before anything is stored (a load behind a store waits for it)
  float4 x = {0.0f, 0.0f, 0.0f, 0.0f}, qv = x;
  if (has) x = Load4(is_v ? rows.v : rows.k, (size_t(s) * g.n_kv + h) * D + d0, rows.dtype);
  if (has && !is_v) qv = Load4(a.q, (size_t(s) * g.n_q + hq) * D + d0, a.q_dtype);  // as the part kernel sees it: f16
  int page = 0, slot = 0;
  if (writes) {  // the token's place: as in the append kernels, position clamped to the table
    const int pos = min(max(a.seq_len[s] - 1, 0), a.stride * g.pt - 1);
    page = ClampPage(a.table[int64_t(s) * a.stride + pos / g.pt], g.n_pages), slot = pos % g.pt;
  }
  uint16_t scale;
  uint32_t own, codes;
  if (g.format == 8) {
    codes = QuantizeLanesQ8(x, &scale), own = codes;
  } else {
    codes = QuantizeLanesQ4(x, lane % 8, &scale, &own);
  }
  const float d = WidenF16(scale);
  float v[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int byte = static_cast<int>((own >> (8 * j)) & 0xFFu);
    v[j] = static_cast<float>(g.format == 8 ? static_cast<int>(static_cast<int8_t>(byte)) : byte - 8) * d;
  }
  if (writes && has) {
    if (g.format == 8) {
      if (is_v) StoreRowV<8>(a.pools, g, page, h, slot, lane, codes, scale);
      else StoreRowK<8>(a.pools, g, page, h, slot, lane, codes, scale);
    } else {
      if (is_v) StoreRowV<4>(a.pools, g, page, h, slot, lane, codes, scale);
      else StoreRowK<4>(a.pools, g, page, h, slot, lane, codes, scale);
    }
  }
  if (is_v) {
    if (has) *reinterpret_cast<float4*>(&vrow[d0]) = float4{v[0], v[1], v[2], v[3]};
    return;
  }
  float dot = static_cast<float>(SaturateToF16(qv.x)) * v[0] + static_cast<float>(SaturateToF16(qv.y)) * v[1] +
              static_cast<float>(SaturateToF16(qv.z)) * v[2] + static_cast<float>(SaturateToF16(qv.w)) * v[3];
  dot = WaveSum(dot);
  if (lane == 0) *score = dot * a.scale;
}

constexpr int kReduceThreads = 256;  // also the number of partial slots weighed at a time (RT below)
constexpr int kReduceThreadsWide = 512;  // ... where a pair has more than that many places for partials
constexpr int kReduceDepth = 4;      // partials a group loads together
constexpr int kReduceMinDims = 32;   // fewest dims of a head one workgroup sums
template <int RT>
__global__ __launch_bounds__(RT) void DattnReduce(const DecodeArgs a, const StepRows rows) {
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv, D = g.hd;
  const int hq = blockIdx.x, s = blockIdx.y, t = threadIdx.x;
  const int h = hq / G, gi = hq % G;
  // this workgroup's dims are [d0, d0 + DZ); the launch's z extent divides a head_dim of 128 or 256: a power of two
  const int DZ = D >> __builtin_ctz(gridDim.z), d0 = blockIdx.z * DZ;
  const size_t o = (size_t(s) * g.n_q + hq) * D + d0;
  const int ts = TilesOf(a, s);
  // the step form: a sequence with a new token has it stored, and (but for the case StepSeesNewToken describes) attended to
  const bool stores_new = rows.k != nullptr && a.seq_len[s] >= 1;
  const bool has_new = stores_new && StepSeesNewToken(a, a.seq_len[s]);
  __shared__ float new_score;
  __shared__ __align__(16) float new_v[256];
  // line units of the sequences before this one and of the whole line; the pair's tiles follow its first units
  size_t p0 = 0, p1 = 0;  // (a sequence that has nothing but its new token has no partials)
  if (ts > 0) {
    // (cut by tile, the sequence is one pair on the line and every head has a row of places of its own)
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
  // The first RT places' (maximum, sum) entries are asked for before the new token's rows are worked on, so the two
  // waits overlap, and stay in registers for the sweep below (a small batch has no more places than that).
  float2 first_ml = {kNegMax, 0.0f};
  if (p0 + t < p1) first_ml = *reinterpret_cast<const float2*>(&a.ml[((p0 + t) * G + gi) * 2]);
  if (stores_new && t < 128) StepToken(a, rows, s, h, hq, t / 64, t % 64, gi == 0 && blockIdx.z == 0, &new_score, new_v);
  if (ts <= 0 && !has_new) {  // nothing to attend to
    for (int d = t; d < DZ; d += RT) a.out[o + d] = 0.0f;
    return;
  }
  constexpr int NW = RT / 64;
  __shared__ float wgt[RT], wl[RT];
  __shared__ int slot[RT];
  __shared__ float red[NW];
  __shared__ int wave_n[NW];
  __shared__ __align__(16) float sums[RT * 4];  // [group][DZ]
  __shared__ float lsums[RT / (kReduceMinDims / 4)];
  // waves that got no tile of this pair left l = 0 (and no acc): they weigh nothing
  float M = first_ml.y > 0.0f ? first_ml.x : kNegMax;
  for (size_t p = p0 + t + RT; p < p1; p += RT)
    if (a.ml[(p * G + gi) * 2 + 1] > 0.0f) M = fmaxf(M, a.ml[(p * G + gi) * 2]);
  M = WaveMax(M);
  if (t % 64 == 0) red[t / 64] = M;
  __syncthreads();
  M = red[0];
  for (int w = 1; w < NW; ++w) M = fmaxf(M, red[w]);
  if (has_new) M = fmaxf(M, new_score);
  const int lg_lanes = __builtin_ctz(static_cast<unsigned>(DZ)) - 2;  // four dims a lane
  const int lanes = 1 << lg_lanes, n_groups = RT >> lg_lanes, grp = t >> lg_lanes, dl = t & (lanes - 1);
  float L = 0.0f;
  float4 A = {0.0f, 0.0f, 0.0f, 0.0f};
  for (size_t b0 = p0; b0 < p1; b0 += RT) {
    const int nb = static_cast<int>(min(p1 - b0, size_t(RT)));
    float l = 0.0f, m = 0.0f;
    if (b0 == p0) l = first_ml.y, m = first_ml.x;
    else if (t < nb) l = a.ml[((b0 + t) * G + gi) * 2 + 1], m = a.ml[((b0 + t) * G + gi) * 2];
    const unsigned long long mask = __ballot(l > 0.0f);
    __syncthreads();  // the previous batch's lists have been read
    if (t % 64 == 0) wave_n[t / 64] = __popcll(mask);
    __syncthreads();
    int at = __popcll(mask & ((1ull << (t % 64)) - 1)), n = 0;  // n: partials of this batch that weigh something
    for (int w = 0; w < NW; ++w) {
      if (w < t / 64) at += wave_n[w];
      n += wave_n[w];
    }
    if (l > 0.0f) {
      const float w = __expf(m - M);
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
    if (has_new) {
      const float w = __expf(new_score - M);
      v = __builtin_fmaf(w, new_v[d0 + d], v), lt += w;
    }
    v /= lt;
    if (a.gate != nullptr) v *= 1.0f / (1.0f + __expf(-a.gate[o + d]));
    a.out[o + d] = v;
  }
}

// ---- host side ----------------------------------------------------------------------------------------------------------


int LaunchPart(const DecodeArgs& a, hipStream_t st) {
  const Geom& m = a.g;
  const dim3 grid(static_cast<unsigned>(a.n_chunks));
  if (a.whole_tiles) {  // (Prepare sets it for q8_0, head_dim 256, 64-token pages and a small batch only)
    hipLaunchKernelGGL(DattnPartWhole, grid, dim3(64 * kWavesPerGroup), 0, st, a);
    return LaunchStatus();
  }
#define YAHKV_LAUNCH_PART(FF, DD, PP)                                                                          \
  do {                                                                                                         \
    if (a.fused) hipLaunchKernelGGL((DattnPart<FF, DD, PP, 1>), grid, dim3(64 * kWavesPerGroup), 0, st, a);           \
    else if (a.wg_partials) hipLaunchKernelGGL((DattnPart<FF, DD, PP, 2>), grid, dim3(64 * kWavesPerGroup), 0, st, a); \
    else hipLaunchKernelGGL((DattnPart<FF, DD, PP, 0>), grid, dim3(64 * kWavesPerGroup), 0, st, a);                    \
  } while (0)
#define YAHKV_LAUNCH_FMT(FF)                                       \
  if (m.hd == 256 && m.pt == 64) YAHKV_LAUNCH_PART(FF, 256, 64);      \
  else if (m.hd == 256 && m.pt == 32) YAHKV_LAUNCH_PART(FF, 256, 32); \
  else if (m.hd == 256) YAHKV_LAUNCH_PART(FF, 256, 16);               \
  else if (m.pt == 64) YAHKV_LAUNCH_PART(FF, 128, 64);                \
  else if (m.pt == 32) YAHKV_LAUNCH_PART(FF, 128, 32);                \
  else YAHKV_LAUNCH_PART(FF, 128, 16)
  if (m.format == 8) {
    YAHKV_LAUNCH_FMT(8);
  } else {
    YAHKV_LAUNCH_FMT(4);
  }
#undef YAHKV_LAUNCH_FMT
#undef YAHKV_LAUNCH_PART
  return LaunchStatus();
}

int LaunchReduce(const DecodeArgs& a, const StepRows& rows, const yahkv_decode_options* opt, hipStream_t st) {
  // a small batch: more workgroups per (query head, sequence), each with a part of the dims, until the CUs have one
  int split = 1;
  while (int64_t(a.g.n_q) * a.n_seqs * split < ComputeUnits() && a.g.hd / (2 * split) >= kReduceMinDims) split *= 2;
  const int asked = MakeTuning(opt).reduce_split;
  if (asked > 0) split = std::min(asked, a.g.hd / kReduceMinDims);
  while (a.g.hd % split != 0 || (a.g.hd / split) % 4 != 0) --split;
  // (a small batch cut into many chunks: a pair's places for partials, eight per chunk its tiles lie in, are weighed in
  // one sweep of a wider workgroup instead of two)
  const int64_t places = int64_t(a.n_chunks) * a.wpc / std::max<int64_t>(int64_t(a.n_seqs) * a.g.n_kv, 1) + a.wpc;
  if (a.wg_partials && places > kReduceThreads)
    hipLaunchKernelGGL(DattnReduce<kReduceThreadsWide>, dim3(a.g.n_q, a.n_seqs, split), dim3(kReduceThreadsWide), 0, st, a, rows);
  else
    hipLaunchKernelGGL(DattnReduce<kReduceThreads>, dim3(a.g.n_q, a.n_seqs, split), dim3(kReduceThreads), 0, st, a, rows);
  return LaunchStatus();
}

int CheckPartArgs(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table, const void* q,
                  int32_t q_dtype) {
  if (const int st = CheckPools(g, pools)) return st;
  if (page_table == nullptr || q == nullptr || (reinterpret_cast<uintptr_t>(q) & 15)) return YAHKV_ERR_ARG;
  if (q_dtype != YAHKV_F32 && q_dtype != YAHKV_F16 && q_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  return YAHKV_OK;
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" size_t yahkv_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                               const yahkv_decode_options* opt) {
  if (CheckGeometry(g) || n_seqs <= 0 || max_seq_len <= 0) return 0;
  return MakePlan(MakeGeom(*g), n_seqs, max_seq_len, MakeTuning(opt)).bytes;
}

extern "C" int yahkv_decode_part(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                 int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                 int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                 void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt,
                                 void* stream) {
  DecodeArgs a;
  if (const int st = CheckGeometry(g)) return st;
  if (const int st = Prepare(MakeGeom(*g), page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, &a))
    return st;
  if (const int st = CheckPartArgs(g, pools, page_table, q, q_dtype)) return st;
  a.pools = MakePools(*pools), a.table = page_table, a.q = q, a.q_dtype = q_dtype, a.scale = softmax_scale;
  return LaunchPart(a, static_cast<hipStream_t>(stream));
}

extern "C" int yahkv_decode_reduce(const yahkv_geometry* g, int32_t page_table_stride, const int32_t* seq_len,
                                   int32_t n_seqs, int32_t max_seq_len, const float* gate, float* out,
                                   const void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt,
                                   void* stream) {
  DecodeArgs a;
  if (const int st = CheckGeometry(g)) return st;
  if (const int st = Prepare(MakeGeom(*g), page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, &a))
    return st;
  if (out == nullptr) return YAHKV_ERR_ARG;
  a.gate = gate, a.out = out;
  return LaunchReduce(a, StepRows{nullptr, nullptr, 0}, opt, static_cast<hipStream_t>(stream));
}

// Append and attention of one decode step in two launches instead of three: the part kernel runs over the tokens the
// pools already hold (lengths one shorter than given), and the reduce quantizes the step's own token, writes it to its
// slot and adds its term to the sums (see StepToken). seq_len[s] counts the new token, which lies at position
// seq_len[s] - 1; a sequence with seq_len[s] <= 0 is left alone (nothing appended, its output rows zero).
extern "C" int yahkv_decode_step_reduce(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                        int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                        int32_t max_seq_len, const void* k_new, const void* v_new, int32_t new_dtype,
                                        const void* q, int32_t q_dtype, float softmax_scale, const float* gate,
                                        float* out, void* workspace, size_t workspace_bytes,
                                        const yahkv_decode_options* opt, void* stream) {
  if (out == nullptr || (reinterpret_cast<uintptr_t>(out) & 15)) return YAHKV_ERR_ARG;
  if (k_new == nullptr || v_new == nullptr) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new)) & 15) return YAHKV_ERR_ARG;
  if (new_dtype != YAHKV_F32 && new_dtype != YAHKV_F16 && new_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if (MakeTuning(opt).one_launch) return YAHKV_ERR_ARG;  // the token enters in the merge's own launch
  DecodeArgs a;
  if (const int st = CheckGeometry(g)) return st;
  if (const int st = Prepare(MakeGeom(*g), page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, &a))
    return st;
  if (const int st = CheckPartArgs(g, pools, page_table, q, q_dtype)) return st;
  a.pools = MakePools(*pools), a.table = page_table, a.q = q, a.q_dtype = q_dtype, a.scale = softmax_scale;
  a.len_bias = -1, a.gate = gate, a.out = out;
  return LaunchReduce(a, StepRows{k_new, v_new, new_dtype}, opt, static_cast<hipStream_t>(stream));
}

extern "C" int yahkv_decode_step(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                 int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                 int32_t max_seq_len, const void* k_new, const void* v_new, int32_t new_dtype,
                                 const void* q, int32_t q_dtype, float softmax_scale, const float* gate, float* out,
                                 void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt,
                                 void* stream) {
  if (out == nullptr || k_new == nullptr || v_new == nullptr) return YAHKV_ERR_ARG;  // before anything is launched
  if ((reinterpret_cast<uintptr_t>(out) | reinterpret_cast<uintptr_t>(k_new) | reinterpret_cast<uintptr_t>(v_new)) & 15)
    return YAHKV_ERR_ARG;
  if (new_dtype != YAHKV_F32 && new_dtype != YAHKV_F16 && new_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if (MakeTuning(opt).one_launch) return YAHKV_ERR_ARG;
  DecodeArgs a;
  if (const int st = CheckGeometry(g)) return st;
  if (const int st = Prepare(MakeGeom(*g), page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, &a))
    return st;
  if (const int st = CheckPartArgs(g, pools, page_table, q, q_dtype)) return st;
  a.pools = MakePools(*pools), a.table = page_table, a.q = q, a.q_dtype = q_dtype, a.scale = softmax_scale;
  a.len_bias = -1;
  if (const int st = LaunchPart(a, static_cast<hipStream_t>(stream))) return st;
  return yahkv_decode_step_reduce(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, k_new, v_new,
                                  new_dtype, q, q_dtype, softmax_scale, gate, out, workspace, workspace_bytes, opt,
                                  stream);
}

namespace yahkv {
namespace {
__global__ void ClearTickets(unsigned long long* tickets, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) tickets[i] = 0ull;
}
}  // namespace
}  // namespace yahkv

// The one-launch form counts arrivals per (sequence, kv head) in the workspace and leaves every count at zero when it
// is done; this call puts the zeros there in the first place (a small fill kernel, so it may be captured into a graph).
extern "C" int yahkv_decode_workspace_init(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                           const yahkv_decode_options* opt, void* workspace, size_t workspace_bytes,
                                           void* stream) {
  if (const int st = CheckGeometry(g)) return st;
  if (workspace == nullptr || (reinterpret_cast<uintptr_t>(workspace) & 15) || n_seqs <= 0 || max_seq_len <= 0)
    return YAHKV_ERR_ARG;
  if (n_seqs > kMaxSeqs) return YAHKV_ERR_SHAPE;
  const Geom m = MakeGeom(*g);
  const Plan p = MakePlan(m, n_seqs, max_seq_len, MakeTuning(opt));
  if (workspace_bytes < p.bytes) return YAHKV_ERR_WORKSPACE;
  const int n = n_seqs * m.n_kv;
  hipLaunchKernelGGL(ClearTickets, dim3((n + 255) / 256), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<unsigned long long*>(static_cast<char*>(workspace) + p.off_tickets), n);
  return LaunchStatus();
}

// Two dispatches, partials and their merge; or, if the caller's options ask for it, one: the split-K kernel, whose
// workgroups then also merge the pairs they are last to finish.
extern "C" int yahkv_decode_attend(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                   int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                   int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                   const float* gate, float* out, void* workspace, size_t workspace_bytes,
                                   const yahkv_decode_options* opt, void* stream) {
  if (out == nullptr || (reinterpret_cast<uintptr_t>(out) & 15)) return YAHKV_ERR_ARG;
  if (!MakeTuning(opt).one_launch) {
    if (const int st = yahkv_decode_part(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q,
                                         q_dtype, softmax_scale, workspace, workspace_bytes, opt, stream))
      return st;
    return yahkv_decode_reduce(g, page_table_stride, seq_len, n_seqs, max_seq_len, gate, out, workspace,
                               workspace_bytes, opt, stream);
  }
  DecodeArgs a;
  if (const int st = CheckGeometry(g)) return st;
  if (const int st = Prepare(MakeGeom(*g), page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, &a))
    return st;
  if (const int st = CheckPartArgs(g, pools, page_table, q, q_dtype)) return st;
  a.pools = MakePools(*pools), a.table = page_table, a.q = q, a.q_dtype = q_dtype, a.scale = softmax_scale;
  a.gate = gate, a.out = out, a.fused = 1;
  return LaunchPart(a, static_cast<hipStream_t>(stream));
}

extern "C" int yahkv_decode_calibrate(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                      int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                      int32_t max_seq_len, const void* q, int32_t q_dtype, void* workspace,
                                      size_t workspace_bytes, yahkv_decode_options* opt, int32_t rounds,
                                      void* stream) {
  hipStream_t st = static_cast<hipStream_t>(stream);
  auto prepare = [&](DecodeArgs* a) -> int {
    if (const int rc = CheckGeometry(g)) return rc;
    if (const int rc = Prepare(MakeGeom(*g), page_table_stride, seq_len, n_seqs, max_seq_len, workspace, workspace_bytes, opt, a))
      return rc;
    if (const int rc = CheckPartArgs(g, pools, page_table, q, q_dtype)) return rc;
    a->pools = MakePools(*pools), a->table = page_table, a->q = q, a->q_dtype = q_dtype, a->scale = 1.0f;
    return YAHKV_OK;
  };
  return CalibrateXcds(prepare, [&](const DecodeArgs& a) { return LaunchPart(a, st); }, workspace, n_seqs, max_seq_len, opt,
                       rounds, st);
}

// ---- the shader clock, as a kernel sees it -----------------------------------------------------------------------------------
//
// One wave counts shader cycles over `ticks` ticks of the constant 100 MHz counter (both counters are the hardware's
// own). What it is for: the instruction-bound kernels here (q4_0 decode, prefill) run as fast as the shader clock, and
// after an idle period the clock is not steady for some tens of milliseconds; a caller that times them can record the
// clock beside each launch (bench.py --clock-trace does).
namespace yahkv {
namespace {
__global__ void ShaderClockProbe(unsigned long long* out, int ticks) {
  if (threadIdx.x != 0) return;
  const unsigned long long w0 = wall_clock64(), c0 = clock64();
  unsigned long long w = w0;
  while (w - w0 < static_cast<unsigned long long>(ticks)) w = wall_clock64();  // the counter always advances
  out[0] = clock64() - c0, out[1] = w - w0;
}
}  // namespace
}  // namespace yahkv

extern "C" int yahkv_shader_clock_probe(void* cycles_and_ticks, int32_t ticks, void* stream) {
  if (cycles_and_ticks == nullptr || (reinterpret_cast<uintptr_t>(cycles_and_ticks) & 7)) return YAHKV_ERR_ARG;
  if (ticks <= 0 || ticks > 100000) return YAHKV_ERR_ARG;  // at most a millisecond
  hipLaunchKernelGGL(ShaderClockProbe, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream),
                     static_cast<unsigned long long*>(cycles_and_ticks), ticks);
  return LaunchStatus();
}

// ---- decode attention without a workspace argument ------------------------------------------------------------------------
//
// For callers that cannot allocate device memory at all (code under HIP graph capture, serving loops or harnesses that
// forbid it): the partials live in an array that is part of the library's code object, so it exists on every GPU the
// library runs on from the moment the code object is loaded there until the process ends. In host code the array's name
// is only a handle for the lookup below; the address the kernels use is the one the runtime reports per device.
constexpr size_t kStaticScratchBytes = size_t(32) << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_of_device[kMaxDevices];  // the array's address on each device, looked up on the first call there

int StaticScratch(void** ptr) {
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return YAHKV_ERR_LAUNCH;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (scratch_of_device[dev] == nullptr) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || p == nullptr) return YAHKV_ERR_LAUNCH;
    scratch_of_device[dev] = p;
  }
  *ptr = scratch_of_device[dev];
  return YAHKV_OK;
}
}  // namespace

extern "C" size_t yahkv_decode_static_scratch_bytes(void) { return kStaticScratchBytes; }

extern "C" int yahkv_decode_attend_static(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                                          int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                                          int32_t max_seq_len, const void* q, int32_t q_dtype, float softmax_scale,
                                          const float* gate, float* out, void* stream) {
  if (const int st = CheckPools(g, pools)) return st;
  if (n_seqs <= 0 || max_seq_len <= 0) return YAHKV_ERR_ARG;
  // the partials of this batch must fit the array: nothing is launched otherwise
  yahkv_decode_options o{};
  o.cut = 1;  // by (sequence, kv head): the cut with the fewest places for partials, so the array holds larger batches
  if (MakePlan(MakeGeom(*g), n_seqs, max_seq_len, MakeTuning(&o)).bytes > kStaticScratchBytes)
    return YAHKV_ERR_WORKSPACE;
  void* ws = nullptr;
  if (const int st = StaticScratch(&ws)) return st;
  return yahkv_decode_attend(g, pools, page_table, page_table_stride, seq_len, n_seqs, max_seq_len, q, q_dtype,
                             softmax_scale, gate, out, ws, kStaticScratchBytes, &o, stream);
}
