// The stream-K cut of the decode attention, shared by the split-K kernels of every pool format: launch arguments,
// the cut of the line of tiles into chunks (ChunkRecord), the walk over a chunk's (sequence, kv head) pairs, the
// partials' places in the workspace, and the host side that sizes the workspace (Plan, Prepare).
#ifndef YAHKV_DECODE_CUT_HPP_
#define YAHKV_DECODE_CUT_HPP_

#include <algorithm>
#include <cstdint>
#include <vector>

#include "common.hpp"

namespace yahkv {

constexpr float kNegMax = -3.4028234663852886e+38f;
constexpr int kTile = 64;     // keys per tile: one wavefront, one key per lane in the score phase
constexpr int kMaxGroup = 8;  // query heads per kv head
constexpr int kMaxSeqs = 8191;
constexpr int kWavesPerGroup = 8;  // one workgroup fills a CU at two waves per SIMD
constexpr int kMergeSlots = 512;   // partial slots the in-kernel merge weighs at a time

struct DecodeArgs {
  Geom g;
  Pools pools;
  const int32_t* table;
  int32_t stride;
  const int32_t* seq_len;
  int32_t n_seqs, max_len;  // max_len: host bound, already clamped to stride * PT
  const void* q;
  int32_t q_dtype;
  float scale;
  const float* gate;
  float* out;
  // workspace
  int32_t* tprefix;  // [n_seqs + 1] line units of all earlier sequences (one kv head's worth); written by part, read by reduce
  float* ml;         // [(n_chunks + n_seqs * H) * wpc][G][2]   partial of (chunk k, wave w, pair p): (k + p) * wpc + w
  float* acc;        // [(n_chunks + n_seqs * H) * wpc][G][D]
  int32_t n_chunks, wpc;  // chunks = workgroups launched; waves per chunk
  int32_t min_chunk_tiles;
  int32_t pair_cost;  // line units a (sequence, kv head) pair takes besides its tiles
  int32_t share[9];  // cumulative shares of the eight chunks of a group, in 1/8192 of the group (share[8] = 8192)
  int32_t deterministic;  // waves take the chunk's tiles in a fixed pattern (the default) instead of first come, first served
  unsigned long long* stamps;  // calibration only: [2 * n_chunks] when each workgroup started, and when its last wave finished
  // one launch for part and merge: the workgroup that is last to finish a pair's tiles merges the pair's partials
  int32_t fused;                // (read by the host, which launches the kernel's one-launch instance)
  int32_t wg_partials;          // (host) the instance that leaves one partial per workgroup for a chunk's last pair
  int32_t whole_tiles;          // (host) ... and asks for a wave's whole tile at once (chunks of about a tile per wave)
  unsigned long long* tickets;  // [n_seqs * H] workgroups that have arrived at a pair's merge; zero between launches
  // The step form (append + attention in two launches): seq_len counts the step's own token, which is not in the
  // pools yet. The part kernel then covers the len_bias = -1 shorter sequences already there, and the reduce
  // quantizes the token's rows, writes them to the pools and adds the token's term to the sums (StepRows).
  int32_t len_bias;
  // Pools whose newest 16-key V tile stays open in f16 (the reference's own format): the split-K kernel covers the
  // closed tiles only, keys 0 .. 16 * ((len - 1) / 16) - 1 whether or not len counts a token still to be appended, and
  // the merge adds the open tile's keys.
  int32_t open_tile;
  // Pools in which the kv heads of a token share rows (the reference's own formats: a token's K scale pairs of all kv
  // heads lie in one row): tile_mult = H cuts the line by (sequence, tile) with the kv heads of a tile next to each
  // other, so that the waves of a workgroup read a row's heads at the same time. A sequence is then one pair of
  // H x tiles items, item j = (tile j / H, kv head j % H). 0 or 1: the line is cut by (sequence, kv head).
  int32_t tile_mult;
};
__device__ __forceinline__ int CutHeads(const DecodeArgs& a) { return a.tile_mult > 1 ? 1 : a.g.n_kv; }
// The step's own token for the reduce kernel: K / V rows [n_seqs][H][D] of `dtype`, or null pointers.
struct StepRows {
  const void* k;
  const void* v;
  int32_t dtype;
};

// Keys of sequence s the part kernel covers. In the step form (len_bias = -1) the length counts a token that is not in
// the pools yet and will go to position len - 1, clamped to the table like every position; the kernel covers what an
// attention after the append would cover, less that token's slot: the slot is the last covered position in every
// case but one (a length beyond the host's bound while the table reaches further: the attention then stops short of
// the new token, as it would after an append of its own).
__device__ __forceinline__ bool StepSeesNewToken(const DecodeArgs& a, int len) {
  const int covered = min(max(len, 0), a.max_len), slot = min(max(len - 1, 0), a.stride * a.g.pt - 1);
  return len >= 1 && slot == covered - 1;
}
__device__ __forceinline__ int ClampLen(const DecodeArgs& a, int s) {
  const int len = a.seq_len[s], covered = min(max(len, 0), a.max_len);
  if (a.open_tile) return covered > 0 ? (covered - 1) & ~15 : 0;
  return a.len_bias != 0 && StepSeesNewToken(a, len) ? covered - 1 : covered;
}

// The line of tiles is cut into groups of eight chunks, 8 A tiles a group; chunk j of a group takes the tiles
// [share[j], share[j + 1]) / 8192 of it. Workgroup k runs on XCD k % 8 and the XCDs do not read memory equally
// fast, so the shares follow their speeds and the workgroups finish together.
__device__ __forceinline__ long long ChunkStart(const DecodeArgs& a, long long A, int k) {
  return (k / 8) * 8 * A + 8 * A * a.share[k % 8] / 8192;
}
__device__ __forceinline__ int ChunkOf(const DecodeArgs& a, long long A, long long tile) {
  const long long span = 8 * A;
  long long group, r;
  if (tile >= 0 && tile < (1ll << 31) && span < (1ll << 31)) {  // one 32-bit division (see ChunkUnits)
    const uint32_t q = static_cast<uint32_t>(tile) / static_cast<uint32_t>(span);
    group = q, r = tile - static_cast<long long>(q) * span;
  } else {
    group = tile / span, r = tile % span;
  }
  int j = 0;
#pragma unroll
  for (int i = 1; i < 8; ++i) j += span * a.share[i] / 8192 <= r;
  return static_cast<int>(group) * 8 + j;
}

// ---- plan -------------------------------------------------------------------------------------------------------------

// The cut of the line is a function of the lengths alone, and every workgroup of the part kernel recomputes its piece
// from them (a few hundred integers from L2) rather than reading the result of a kernel of its own: a dispatch
// between the append and the attention costs more than all these recomputations together. The first workgroup
// leaves the prefix sums in the workspace for the reduce, which needs two of them per workgroup.
//
// The line is measured in units of one tile's work. A pair (sequence, kv head) of ts tiles takes pair_cost + ts units:
// first the units that stand for what a change of pair costs every wave of a workgroup (it drains its pipeline,
// leaves a partial and fetches new queries: about eight tiles' worth per workgroup, measured), then one unit per
// tile. Cutting this line evenly gives chunks of equal time rather than of equal tiles: without it the workgroups
// finish up to 50 us apart, by the number of pairs their chunks hold.
__device__ __forceinline__ int TilesOf(const DecodeArgs& a, int s) {
  return (ClampLen(a, s) + kTile - 1) / kTile * max(a.tile_mult, 1);
}
__device__ __forceinline__ int UnitsOf(const DecodeArgs& a, int ts) { return ts > 0 ? ts + a.pair_cost : 0; }
// (Divisions of line coordinates: 64-bit divisions by run-time values are long sequences of scalar instructions, which
// every wave of the merge kernel would repeat; a line below 2^31 units, any real one, takes the 32-bit form.)
__device__ __forceinline__ long long ChunkUnits(const DecodeArgs& a, long long line) {
  // a short line is not cut finer than min_chunk_tiles: each piece costs a partial (G x (D + 2) floats)
  const long long per = line < (1ll << 31) - (1 << 21)
                            ? static_cast<long long>((static_cast<uint32_t>(line) + static_cast<uint32_t>(a.n_chunks) - 1u) /
                                                     static_cast<uint32_t>(a.n_chunks))
                            : (line + a.n_chunks - 1) / a.n_chunks;
  return max(per, static_cast<long long>(a.min_chunk_tiles));
}

// Chunk k of the line, for a whole workgroup of NT threads (all call it; two barriers inside): {sequence or -1, kv
// head, first tile within the pair, tiles in the chunk}. Thread t sums a slice of the sequences, a scan over the
// threads gives every slice its place on the line, and the threads whose slices hold the chunk's two ends walk
// their slices to find the sequences and count the tiles before each end.
// Also leaves, for the merge: tiles_at[2], the line coordinate of the first tile of the chunk's first pair, and
// tiles_at[3], the line units per chunk (the A of ChunkStart / ChunkOf).
template <int NT>
__device__ __forceinline__ int4 ChunkRecord(const DecodeArgs& a, int k, int (*wave_sum)[2], int4* found, long long* tiles_at,
                                            bool* any_empty) {
  const int t = threadIdx.x, H = CutHeads(a), c = a.pair_cost;
  const int per = (a.n_seqs + NT - 1) / NT;
  const int s0 = min(t * per, a.n_seqs), s1 = min(s0 + per, a.n_seqs);
  int sum = 0, cnt = 0;  // units of the slice, and sequences in it that are not empty
  for (int s = s0; s < s1; ++s) {
    const int ts = TilesOf(a, s);
    sum += UnitsOf(a, ts), cnt += ts > 0;
  }
  *any_empty = cnt < s1 - s0;
  int incl = sum, incl_cnt = cnt;  // inclusive scans inside the wave, then the waves' totals
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(incl, o, 64), vc = __shfl_up(incl_cnt, o, 64);
    if (t % 64 >= o) incl += v, incl_cnt += vc;
  }
  if (t % 64 == 63) wave_sum[t / 64][0] = incl, wave_sum[t / 64][1] = incl_cnt;
  __syncthreads();
  int base = incl - sum, base_cnt = incl_cnt - cnt, total = 0, total_cnt = 0;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) {
    if (w < t / 64) base += wave_sum[w][0], base_cnt += wave_sum[w][1];
    total += wave_sum[w][0], total_cnt += wave_sum[w][1];
  }
  if (k == 0) {
    int before = base;
    for (int s = s0; s < s1; ++s) a.tprefix[s] = before, before += UnitsOf(a, TilesOf(a, s));
    if (t == 0) a.tprefix[a.n_seqs] = total;
  }
  const long long line = static_cast<long long>(total) * H, A = ChunkUnits(a, line);
  if (t == 0) tiles_at[3] = A;
  const long long start = ChunkStart(a, A, k), end = min(ChunkStart(a, A, k + 1), line);
  if (start >= end) return int4{-1, 0, 0, 0};  // the same for every thread
  if (t == 0 && end == line) tiles_at[1] = static_cast<long long>(total - c * total_cnt) * H;
  // tiles before line position x, and where x lies, for the thread whose slice holds x
  auto locate = [&](long long x, int4* where, long long* tiles) {
    if (x < static_cast<long long>(base) * H || x >= static_cast<long long>(base + sum) * H) return;
    int before = base, before_cnt = base_cnt;
    for (int s = s0; s < s1; ++s) {
      const int ts = TilesOf(a, s), units = UnitsOf(a, ts);
      if (x < static_cast<long long>(before + units) * H) {
        const int r = static_cast<int>(x - static_cast<long long>(before) * H);
        const int h = r / units, first = max(r % units - c, 0);
        *tiles = static_cast<long long>(before - c * before_cnt) * H + static_cast<long long>(h) * ts + first;
        if (where != nullptr) {
          *where = int4{s, h, first, 0};
          tiles_at[2] = static_cast<long long>(before) * H + static_cast<long long>(h) * units + c;
        }
        return;
      }
      before += units, before_cnt += ts > 0;
    }
  };
  locate(start, found, &tiles_at[0]);
  if (end < line) locate(end, nullptr, &tiles_at[1]);
  __syncthreads();
  int4 rec = *found;
  rec.w = static_cast<int>(tiles_at[1] - tiles_at[0]);
  if (rec.w <= 0) return int4{-1, 0, 0, 0};  // the chunk lies inside a pair's first units
  return rec;
}

// The same record for a batch of at most 64 sequences, computed by every wave for itself (lane = sequence): no LDS,
// no barrier, one load per lane and a handful of shuffles, where the general form costs two barriers and a loop per
// thread. A small batch is where this matters: its part kernel runs some tens of microseconds, and the cut is a
// dependent prologue in front of every wave's first load. The first wave of the workgroup leaves the record in LDS for
// the merge at the kernel's end (which reads it behind a barrier).
__device__ __forceinline__ int4 ChunkRecordWave(const DecodeArgs& a, int k, int wave, int lane, int4* found, long long* tiles_at,
                                                bool* any_empty) {
  const int H = CutHeads(a), c = a.pair_cost;
  const int ts = lane < a.n_seqs ? TilesOf(a, lane) : 0, units = UnitsOf(a, ts), cnt = ts > 0;
  *any_empty = __builtin_amdgcn_ballot_w64(lane < a.n_seqs && ts == 0) != 0;
  int incl = units, incl_cnt = cnt;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(incl, o, 64), vc = __shfl_up(incl_cnt, o, 64);
    if (lane >= o) incl += v, incl_cnt += vc;
  }
  const int base = incl - units, base_cnt = incl_cnt - cnt;
  const int total = __shfl(incl, 63, 64), total_cnt = __shfl(incl_cnt, 63, 64);
  if (k == 0 && wave == 0) {
    if (lane < a.n_seqs) a.tprefix[lane] = base;
    if (lane == 0) a.tprefix[a.n_seqs] = total;
  }
  const long long line = static_cast<long long>(total) * H, A = ChunkUnits(a, line);
  const long long start = ChunkStart(a, A, k), end = min(ChunkStart(a, A, k + 1), line);
  if (start >= end) return int4{-1, 0, 0, 0};
  // where line position x lies: the lane (sequence) whose stretch holds it works it out, the others take its answer
  auto locate = [&](long long x, int* s_, int* h_, int* first_, long long* tiles, long long* line0) {
    const bool mine = units > 0 && x >= static_cast<long long>(base) * H && x < static_cast<long long>(base + units) * H;
    const int src = __builtin_ctzll(__builtin_amdgcn_ballot_w64(mine) | (1ull << 63));
    const int r = static_cast<int>(x - static_cast<long long>(base) * H);
    const int h = mine ? r / units : 0, first = mine ? max(r % units - c, 0) : 0;
    const long long t = static_cast<long long>(base - c * base_cnt) * H + static_cast<long long>(h) * ts + first;
    const long long l0 = static_cast<long long>(base) * H + static_cast<long long>(h) * units + c;
    *s_ = src, *h_ = __shfl(h, src, 64), *first_ = __shfl(first, src, 64);
    *tiles = __shfl(t, src, 64), *line0 = __shfl(l0, src, 64);
  };
  int s0, h0, f0, s1, h1, f1;
  long long t0, t1, l0, l1;
  locate(start, &s0, &h0, &f0, &t0, &l0);
  if (end < line) locate(end, &s1, &h1, &f1, &t1, &l1);
  else t1 = static_cast<long long>(total - c * total_cnt) * H;
  int4 rec = {s0, h0, f0, static_cast<int>(t1 - t0)};
  if (wave == 0 && lane == 0) *found = rec, tiles_at[0] = t0, tiles_at[1] = t1, tiles_at[2] = l0, tiles_at[3] = A;
  if (rec.w <= 0) return int4{-1, 0, 0, 0};
  return rec;
}

// Position of a wave on its chunk: the pair (s, h) it stands on, which of the chunk's tiles belong to that pair
// ([base, base + n) in chunk numbering, starting at the pair's tile `first`), and that sequence's length.
struct PairCursor {
  int s, h, first, base, n, len;
};
__device__ __forceinline__ PairCursor FirstPair(const DecodeArgs& a, const int4 rec) {
  const int ts = TilesOf(a, rec.x);
  return PairCursor{rec.x, rec.y, rec.z, 0, min(ts - rec.z, rec.w), ClampLen(a, rec.x)};
}
// Next pair of the chunk; false when the chunk (of chunk_n tiles) ends with the current pair.
__device__ __forceinline__ bool NextPair(const DecodeArgs& a, int chunk_n, PairCursor* c) {
  if (c->base + c->n >= chunk_n) return false;
  c->base += c->n, c->first = 0;
  int ts = 0;
  do {  // empty sequences have no tiles on the line
    if (++c->h == CutHeads(a)) c->h = 0, ++c->s;
    if (c->s >= a.n_seqs) return false;
    ts = TilesOf(a, c->s);
    if (ts == 0) c->h = CutHeads(a) - 1;
  } while (ts == 0);
  c->n = min(ts, chunk_n - c->base), c->len = ClampLen(a, c->s);
  return true;
}
// The same walk for the merge at the kernel's end, which also needs to know where on the line a pair lies: its tiles
// in all and the line coordinate of its first tile.
struct MergeCursor {
  PairCursor c;
  int ts;
  long long line0;
};
__device__ __forceinline__ MergeCursor FirstMergePair(const DecodeArgs& a, const int4 rec, long long line0) {
  return MergeCursor{FirstPair(a, rec), TilesOf(a, rec.x), line0};
}
__device__ __forceinline__ bool NextMergePair(const DecodeArgs& a, int chunk_n, MergeCursor* m) {
  const long long next = m->line0 + m->ts + a.pair_cost;  // the next pair's first units follow this pair's tiles
  if (!NextPair(a, chunk_n, &m->c)) return false;         // (sequences without keys take none)
  m->line0 = next, m->ts = TilesOf(a, m->c.s);
  return true;
}
__device__ __forceinline__ size_t PartialIndex(const DecodeArgs& a, int chunk, int wave, const PairCursor& c) {
  return (size_t(chunk) + size_t(c.s) * a.g.n_kv + c.h) * a.wpc + wave;
}

// ---- shared pieces ----------------------------------------------------------------------------------------------------

__device__ __forceinline__ float WaveMax(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float HalfMax32(float v) {  // over the 32 lanes of a wave half
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float HalfSum32(float v) {
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

typedef _Float16 h2v __attribute__((ext_vector_type(2)));
typedef _Float16 h8v __attribute__((ext_vector_type(8)));
typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

// Eight consecutive query elements as f16. f16 sources are taken as they are; bf16 sources convert exactly in the
// normal f16 range, f32 sources (what the reference's kernels take, gen_decode_attn.py:576) round to nearest even;
// finite values beyond the f16 range saturate at +-65504 instead of becoming infinite (an infinite score would turn the
// whole row into NaN); NaN and infinite inputs give NaN.
__device__ __forceinline__ _Float16 SaturateToF16(float x) {
  return static_cast<_Float16>(__builtin_fminf(__builtin_fmaxf(x, -65504.0f), 65504.0f) + (x - x));  // x - x: 0, or NaN
}
// Eight query elements in two steps, so that a kernel can ask for them, ask for other things, and only then wait: the
// bytes as they lie in memory (f32: 32 of them, f16 / bf16: 16), and their f16 values.
struct RawQ8 {
  uint4 a, b;
};
__device__ __forceinline__ RawQ8 LoadRawQ8(const void* q, size_t i, int dt) {
  RawQ8 r;
  if (dt == YAHKV_F32) {
    r.a = *reinterpret_cast<const uint4*>(static_cast<const float*>(q) + i);
    r.b = *reinterpret_cast<const uint4*>(static_cast<const float*>(q) + i + 4);
  } else {
    r.a = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(q) + i);
    r.b = uint4{0u, 0u, 0u, 0u};
  }
  return r;
}
__device__ __forceinline__ h8v ConvertQ8(const RawQ8& raw, int dt) {
  h8v r;
  if (dt == YAHKV_F32) {
    const uint32_t v[8] = {raw.a.x, raw.a.y, raw.a.z, raw.a.w, raw.b.x, raw.b.y, raw.b.z, raw.b.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = SaturateToF16(__builtin_bit_cast(float, v[j]));
  } else {
    const uint32_t w[4] = {raw.a.x, raw.a.y, raw.a.z, raw.a.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const uint16_t hbits = static_cast<uint16_t>(w[j / 2] >> (16 * (j % 2)));
      r[j] = dt == YAHKV_F16 ? __builtin_bit_cast(_Float16, hbits) : SaturateToF16(WidenBf16(hbits));
    }
  }
  return r;
}
__device__ __forceinline__ h8v LoadQ8(const void* q, size_t i, int dt) { return ConvertQ8(LoadRawQ8(q, i, dt), dt); }

// Partials travel between workgroups on different XCDs, whose L2 caches do not see each other's lines: they are
// written through to memory and read past the L2 (cache policy sc1, device scope) by these buffer accesses. Fences of
// device scope would do it too, but they write back and invalidate a whole L2, and with it the K / V lines the XCD's
// other workgroups have in flight (measured: 12 % of the kernel's time).
constexpr int kDeviceScope = 16;  // the sc1 bit of a buffer instruction's cache policy
typedef unsigned int u4v __attribute__((__vector_size__(4 * sizeof(unsigned int))));
typedef unsigned int u2v __attribute__((__vector_size__(2 * sizeof(unsigned int))));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t DeviceBuffer(const void* base) {  // base: the same in every lane
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, 0x7fffffff, 0x00020000);
}
__device__ __forceinline__ void StoreDevice(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, float v) {
  __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned int, v), r, byte_offset, 0, kDeviceScope);
}
__device__ __forceinline__ void StoreDevice2(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset, float x, float y) {
  const u2v w = {__builtin_bit_cast(unsigned int, x), __builtin_bit_cast(unsigned int, y)};
  __builtin_amdgcn_raw_buffer_store_b64(w, r, byte_offset, 0, kDeviceScope);
}
__device__ __forceinline__ float2 LoadDevice2(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset) {
  const u2v w = __builtin_amdgcn_raw_buffer_load_b64(r, byte_offset, 0, kDeviceScope);
  const unsigned int w0 = w[0], w1 = w[1];  // (a bit cast applied to w[1] directly reads w[0] with this compiler)
  return float2{__builtin_bit_cast(float, w0), __builtin_bit_cast(float, w1)};
}
template <int N>
struct LoadDeviceN;
template <>
struct LoadDeviceN<4> {
  typedef float type __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset) {
    return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b128(r, byte_offset, 0, kDeviceScope));
  }
};
template <>
struct LoadDeviceN<2> {
  typedef float type __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ type load(__amdgpu_buffer_rsrc_t r, uint32_t byte_offset) {
    return __builtin_bit_cast(type, __builtin_amdgcn_raw_buffer_load_b64(r, byte_offset, 0, kDeviceScope));
  }
};

// Workspace layout and chunk count, from the host's bounds alone (the lengths are on the device).
struct Plan {
  int32_t max_len, n_chunks, wpc, min_chunk_tiles, pair_cost;
  int32_t share[9];
  size_t off_tprefix, off_tickets, off_ml, off_acc, off_stamps, bytes;
};
inline size_t Align(size_t x) { return (x + 255) & ~size_t(255); }
inline int ComputeUnits() {
  static const int cus = [] {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    return n;
  }();
  return cus;
}
// Tuning values of a call: the caller's options where given, else the defaults.
struct Tuning {
  int32_t n_chunks, min_chunk_tiles, pair_cost, reduce_split, deterministic, one_launch, wg_partials, cut;
  bool min_chunk_given, pair_cost_given;
  int32_t xcd_weight[8];
};
inline Tuning MakeTuning(const yahkv_decode_options* o) {
  Tuning t{};
  // one 8-wave workgroup per CU (two waves per SIMD)
  t.n_chunks = o != nullptr && o->n_chunks > 0 ? std::min(o->n_chunks, 1 << 20) : ComputeUnits();
  // at least 2: with chunks of one unit the smaller shares of a group of eight would round to nothing, and the merge
  // counts on every chunk inside a pair's stretch of the line having left partials
  t.min_chunk_tiles = o != nullptr && o->min_chunk_tiles > 0 ? std::min(std::max(o->min_chunk_tiles, 2), 1 << 20)
                                                             : 2 * kWavesPerGroup;
  t.min_chunk_given = o != nullptr && o->min_chunk_tiles > 0;
  t.pair_cost_given = o != nullptr && o->pair_cost != 0;
  t.pair_cost = o == nullptr || o->pair_cost == 0 ? 8 : std::min(std::max(o->pair_cost, 0), 1 << 10);
  t.reduce_split = o != nullptr ? std::max(o->reduce_split, 0) : 0;
  t.deterministic = o == nullptr || o->deterministic >= 0;  // (negative: tiles first come, first served)
  t.one_launch = o != nullptr && o->one_launch != 0;
  t.wg_partials = o != nullptr ? o->wg_partials : 0;
  t.cut = o != nullptr ? o->cut : 0;
  for (int j = 0; j < 8; ++j) t.xcd_weight[j] = o != nullptr ? std::max(o->xcd_weight[j], 0) : 0;
  return t;
}
// Whether the line is cut by (sequence, tile), DecodeArgs::tile_mult: the reference's own formats wherever the kv head
// count allows it, the block formats when the options ask for it.
inline bool CutByTile(const Geom& g, const Tuning& t) {
  if (g.n_kv <= 1 || kWavesPerGroup % g.n_kv != 0) return false;
  return g.format > 16 || (t.cut != 1 && !t.one_launch && t.wg_partials != 1);
}
// Whether a batch is small enough for whole-tile requests (DattnPart's MODE 3: q8_0, head_dim 256, a tile = a page): at
// most two tiles per wave when every CU has a workgroup. Such a batch is cut into chunks of one tile per wave.
inline bool WholeTiles(const Geom& g, const Tuning& t, int64_t line_max) {
  return g.format == 8 && g.hd == 256 && g.pt == kTile && !t.one_launch && (t.wg_partials == 0 || t.wg_partials == 3) &&
         line_max <= int64_t(t.n_chunks) * kWavesPerGroup * 2;
}
inline Plan MakePlan(const Geom& g, int32_t n_seqs, int32_t max_seq_len, const Tuning& t) {
  Plan p;
  p.max_len = std::max(max_seq_len, 1);
  const int64_t max_tiles = (int64_t(p.max_len) + kTile - 1) / kTile;
  const int64_t line_max = max_tiles * n_seqs * g.n_kv;
  p.wpc = kWavesPerGroup;
  p.min_chunk_tiles = t.min_chunk_tiles, p.pair_cost = t.pair_cost;
  if (WholeTiles(g, t, line_max)) {  // one tile per wave wherever the line allows it: a pair costs nothing besides
    if (!t.min_chunk_given) p.min_chunk_tiles = kWavesPerGroup;
    if (!t.pair_cost_given) p.pair_cost = 0;
  }
  p.n_chunks =
      static_cast<int32_t>(std::min<int64_t>(t.n_chunks, (line_max + p.min_chunk_tiles - 1) / p.min_chunk_tiles));
  // Shares of the eight chunks of a group: proportional to the caller's relative XCD speeds (yahkv_decode_calibrate
  // measures them), equal without them. No share falls below 1 / 16 of the group, which at two line units per chunk is
  // one unit: no chunk inside a pair's stretch comes out empty. (Shares below that bound are raised to it and the rest
  // is dealt out again among the others.)
  double w[8], share[8];
  double sum = 0;
  for (int j = 0; j < 8; ++j) w[j] = t.xcd_weight[j], sum += w[j];
  // (a last group that is not whole would leave the line's end uncovered: equal shares then)
  if (sum <= 0 || p.n_chunks % 8 != 0) std::fill(w, w + 8, 1.0);
  bool low[8] = {false, false, false, false, false, false, false, false};
  for (int round = 0; round < 8; ++round) {
    double free_sum = 0, left = 8192;
    for (int j = 0; j < 8; ++j) low[j] ? left -= 512 : free_sum += w[j];
    bool again = false;
    for (int j = 0; j < 8; ++j) {
      share[j] = low[j] || free_sum <= 0 ? 512 : w[j] * left / free_sum;
      if (share[j] < 512) low[j] = again = true;
    }
    if (!again) break;
  }
  p.share[0] = 0;
  for (int j = 0; j < 8; ++j) p.share[j + 1] = p.share[j] + std::max(512, static_cast<int32_t>(share[j]));
  // rounding leaves a few 8192ths over or short: the last chunks take them, none going below its bound
  for (int j = 8, over = p.share[8] - 8192; j >= 1; --j) p.share[j] = std::min(p.share[j] - over, 8192 - 512 * (8 - j));
  p.share[8] = 8192;
  // (the formats whose line is cut by (sequence, tile), DecodeArgs::tile_mult, keep a row of places per kv head)
  const bool by_tile = CutByTile(g, t);
  const size_t parts = (by_tile ? (size_t(p.n_chunks) + size_t(n_seqs)) * g.n_kv : size_t(p.n_chunks) + size_t(n_seqs) * g.n_kv) * p.wpc;
  p.off_tprefix = 0;
  p.off_tickets = Align(sizeof(int32_t) * (size_t(n_seqs) + 1));
  p.off_ml = Align(p.off_tickets + sizeof(unsigned long long) * size_t(n_seqs) * g.n_kv);
  p.off_acc = Align(p.off_ml + sizeof(float) * parts * g.group() * 2);
  p.off_stamps = Align(p.off_acc + sizeof(float) * parts * g.group() * g.hd);  // for yahkv_decode_calibrate
  p.bytes = Align(p.off_stamps + 2 * sizeof(unsigned long long) * size_t(p.n_chunks));
  return p;
}

// Fills the launch arguments all dispatches share; returns a status. `m`: a geometry the caller has validated (the
// formats have their own checks).
inline int Prepare(const Geom& m, int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                   const void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt, DecodeArgs* a) {
  if (seq_len == nullptr || workspace == nullptr) return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || max_seq_len <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (n_seqs > kMaxSeqs) return YAHKV_ERR_SHAPE;  // every workgroup walks all lengths: keep that a few thousand
  if (reinterpret_cast<uintptr_t>(workspace) & 15) return YAHKV_ERR_ARG;
  const Tuning t = MakeTuning(opt);
  const Plan p = MakePlan(m, n_seqs, max_seq_len, t);
  if (workspace_bytes < p.bytes) return YAHKV_ERR_WORKSPACE;
  *a = DecodeArgs{};
  a->g = m, a->stride = page_table_stride, a->seq_len = seq_len, a->n_seqs = n_seqs;
  // lengths read on the device are clamped to the host's bound and to the table's extent
  a->max_len = static_cast<int32_t>(std::min<int64_t>(p.max_len, int64_t(page_table_stride) * m.pt));
  char* ws = static_cast<char*>(const_cast<void*>(workspace));
  a->tprefix = reinterpret_cast<int32_t*>(ws + p.off_tprefix);
  a->tickets = reinterpret_cast<unsigned long long*>(ws + p.off_tickets);
  a->ml = reinterpret_cast<float*>(ws + p.off_ml);
  a->acc = reinterpret_cast<float*>(ws + p.off_acc);
  a->n_chunks = p.n_chunks, a->wpc = p.wpc, a->min_chunk_tiles = p.min_chunk_tiles, a->pair_cost = p.pair_cost;
  a->deterministic = t.deterministic;
  // One partial per workgroup for a chunk's last pair pays where chunks are short (a small batch: few tiles per wave, so
  // a wave's partial is a large part of what it moves) and costs two barriers at the kernel's end where they are long.
  a->wg_partials = t.wg_partials == 1 || t.wg_partials == 3 ? 1 : t.wg_partials == 2 ? 0 : (int64_t(p.max_len) + kTile - 1) / kTile * n_seqs * m.n_kv <= int64_t(p.n_chunks) * kWavesPerGroup * 4;
  a->whole_tiles = a->wg_partials && WholeTiles(m, t, (int64_t(p.max_len) + kTile - 1) / kTile * n_seqs * m.n_kv);
  if (m.format <= 16 && CutByTile(m, t) && !a->wg_partials) a->tile_mult = m.n_kv;
  std::copy(p.share, p.share + 9, a->share);
  return YAHKV_OK;
}

// ---- XCD calibration -----------------------------------------------------------------------------------------------------

constexpr int kCalibrationLaunches = 8;  // measured launches per round

// Relative read speeds of the eight XCDs on the caller's own batch. Workgroup k of a dispatch runs on XCD k % 8, and the
// XCDs of one GPU do not read memory equally fast (up to 10 % apart, measured); chunk shares that follow their speeds
// let all workgroups finish together. Each round (`rounds` of them, and one more that only measures) runs the part
// kernel nine times with the current shares (the first launch warms caches and clocks), reads when each workgroup's last wave finished, and sets every XCD's weight to its
// share divided by its mean time over the eight measured launches. The XCDs read the same memory, so what one of them
// gives up the others partly take: a round corrects about half of what it sees, and a later round can overshoot (the
// calibration's own launches on a ragged batch of 64: 801 us with equal shares, 782 after three rounds, 771 - 776 from
// the fourth on, up and down by a few us). Every round therefore also notes how long the launches took with the weights
// it was given, and the call ends on the weights that were measured fastest, not on the last ones computed. (Steps
// timed afterwards are 0.5 % shorter after three rounds than after one, and no shorter after eight.) Synchronizes the
// stream: a set-up call, not part of a step.
// `prepare` fills the launch arguments from the caller's (and validates them), `launch` runs the part kernel.
template <typename PrepareFn, typename LaunchFn>
inline int CalibrateXcds(PrepareFn prepare, LaunchFn launch, void* workspace, int32_t n_seqs, int32_t max_seq_len,
                         yahkv_decode_options* opt, int32_t rounds, hipStream_t st) {
  if (opt == nullptr || rounds <= 0) return YAHKV_ERR_ARG;
  int32_t best_weight[8];
  double best_span = -1.0;
  auto keep_best = [&]() {
    if (best_span < 0) return;
    std::copy(best_weight, best_weight + 8, opt->xcd_weight);
    // (equal shares, if the caller's all-zero weights were the fastest, are written as such: the weights then say that
    // a calibration has run)
    if (std::all_of(best_weight, best_weight + 8, [](int32_t w) { return w == 0; })) std::fill(opt->xcd_weight, opt->xcd_weight + 8, 10000);
  };
  for (int32_t r = 0; r <= rounds; ++r) {  // (the round after the last only measures what the last one computed)
    DecodeArgs a;
    if (const int rc = prepare(&a)) return rc;
    if (a.n_chunks % 8 != 0) return YAHKV_OK;  // a batch too small for whole groups is cut into equal shares anyway
    const Plan p = MakePlan(a.g, n_seqs, max_seq_len, MakeTuning(opt));
    a.stamps = reinterpret_cast<unsigned long long*>(static_cast<char*>(workspace) + p.off_stamps);
    const size_t n = 2 * size_t(a.n_chunks);  // [0, n_chunks): start of each workgroup, [n_chunks, ..): its end
    std::vector<unsigned long long> stamps(n);
    double t[8] = {0, 0, 0, 0, 0, 0, 0, 0}, span = 0;
    int cnt[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int pass = 0; pass < 1 + kCalibrationLaunches; ++pass) {  // the first launch warms caches and clocks
      if (hipMemsetAsync(a.stamps, 0, n * sizeof(unsigned long long), st) != hipSuccess) return YAHKV_ERR_LAUNCH;
      if (const int rc = launch(a)) return rc;
      if (pass == 0) continue;
      if (hipMemcpyAsync(stamps.data(), a.stamps, n * sizeof(unsigned long long), hipMemcpyDeviceToHost, st) != hipSuccess ||
          hipStreamSynchronize(st) != hipSuccess)
        return YAHKV_ERR_LAUNCH;
      unsigned long long start = ~0ull;
      for (int k = 0; k < a.n_chunks; ++k)
        if (stamps[size_t(k)] != 0) start = std::min(start, stamps[size_t(k)]);
      unsigned long long last = start;
      for (int k = 0; k < a.n_chunks; ++k) {
        const unsigned long long end = stamps[size_t(a.n_chunks) + size_t(k)];
        if (end > start) t[k % 8] += double(end - start), ++cnt[k % 8];
        last = std::max(last, end);
      }
      span += double(last - start);
    }
    if (best_span < 0 || span < best_span) {  // the weights this round was given, and what the launches took with them
      best_span = span;
      std::copy(opt->xcd_weight, opt->xcd_weight + 8, best_weight);
    }
    if (r == rounds) break;
    double speed[8], top = 0;
    for (int j = 0; j < 8; ++j) {
      if (cnt[j] == 0 || t[j] <= 0) {  // an XCD without work: nothing to learn from this batch
        keep_best();
        return YAHKV_OK;
      }
      speed[j] = double(a.share[j + 1] - a.share[j]) / (t[j] / cnt[j]);
      top = std::max(top, speed[j]);
    }
    for (int j = 0; j < 8; ++j) opt->xcd_weight[j] = std::max(1, static_cast<int32_t>(speed[j] / top * 10000.0 + 0.5));
  }
  keep_best();
  return YAHKV_OK;
}

}  // namespace yahkv

#endif  // YAHKV_DECODE_CUT_HPP_
