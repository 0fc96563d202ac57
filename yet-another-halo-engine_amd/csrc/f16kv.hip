// The reference's unquantized twins of the decode path: yah_dattn_kvappend (gen_decode_attn.py:30-94), yah_dattn_part
// (:97-335) and yah_dattn_reduce (:338-411) on pools of f16 K and f16 V^T, through the same page table, positions and
// clamping as the quantized kernels. A first, plain version: no software pipeline, a fixed split of every sequence.
//
// Pool layouts, per page and kv head (elements are f16):
//   K    [D / 16][PT][16]   a lane's 16-byte load is 8 dims of one key; the 32 keys of a tile are 1 KB per 16-dim group
//   V^T  [PT / R][D][R]      in runs of R = min(PT, 32) keys; a lane's 16-byte load is 8 keys of one dim
// Both products run on the matrix cores in f16 with f32 accumulation, as in the quantized kernel: scores
// S[head][key] with v_mfma_f32_32x32x16_f16 (queries as A rows, 8 of 32 rows used), O[head][dim] += P V with
// v_mfma_f32_16x16x32_f16 (P rounded to f16 against the running maximum).
#include <algorithm>
#include <cstdlib>

#include "common.hpp"
#include "decode_cut.hpp"

namespace yahkv {
namespace {

typedef float f4v __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr int kTileKeys = 32;   // keys per tile (one wave, one pass)
constexpr int kWaves = 4;       // waves per workgroup; they take the tiles of the workgroup's stretch in turn
constexpr int kMaxHeads = 8;    // query heads per kv head
constexpr int kRunAppendMinTokens = 8;  // chunks of at least this many tokens per sequence go run by run
constexpr float kLowest = -3.4028234663852886e+38f;
constexpr float kLog2e = 1.4426950408889634f, kLn2 = 0.6931471805599453f;

struct F16Args {
  Geom g;
  uint16_t* k;
  uint16_t* v;
  const int32_t* table;
  int32_t stride;
  // append
  const int32_t* start_pos;
  const int32_t* n_valid;
  int32_t n_seqs, n_new;
  const void* k_src;
  const void* v_src;
  int32_t src_dtype;
  // decode
  const int32_t* seq_len;
  int32_t max_len;
  const void* q;
  int32_t q_dtype;
  float scale;
  float* ml;   // [n_seqs][H][n_splits][G][2]: running maximum (natural-log units) and sum of a stretch
  float* acc;  // [n_seqs][H][n_splits][G][D]
  int32_t n_splits, keys_per_split;
  const float* gate;
  float* out;
};

__device__ __forceinline__ size_t KOffset(const Geom& g, size_t page_head, int dim, int t) {
  return (page_head * (g.hd / 16) + dim / 16) * (size_t(g.pt) * 16) + size_t(t) * 16 + dim % 16;
}
// V^T in runs of at most 32 keys: the 32 keys that one wave takes at a time are whole 64-byte rows of one 16 KB
// block then, where rows of 64 keys would leave every 128-byte line to two waves at different times.
__device__ __forceinline__ size_t VOffset(const Geom& g, size_t page_head, int dim, int t) {
  const int run = min(g.pt, 32);
  return page_head * (size_t(g.hd) * g.pt) + (size_t(t / run) * g.hd + dim) * run + t % run;
}

// One thread per (token, kv head, dim): K and V of that element, rounded to f16 (round to nearest even: the
// reference's fptrunc, gen_decode_attn.py:79-80), at the token's page row. Positions clamp to the table as
// everywhere (:59-63); where several tokens of a chunk clamp to one slot the last wins, as in a loop over the tokens.
__global__ __launch_bounds__(256) void AppendF16(const F16Args a) {
  const Geom g = a.g;
  const int H = g.n_kv, PT = g.pt, D = g.hd;
  const int i = blockIdx.x, h = blockIdx.y, s = blockIdx.z, d = threadIdx.x;
  const int nv = a.n_valid != nullptr ? min(max(a.n_valid[s], 0), a.n_new) : a.n_new;
  if (i >= nv || d >= D) return;
  const int start = a.start_pos[s], last_pos = a.stride * PT - 1;
  const int pos = min(max(start + i, 0), last_pos);
  int winner = pos - start;  // the token of the chunk that ends up at pos
  if (pos == last_pos && start + nv - 1 >= last_pos) winner = nv - 1;
  if (pos == 0 && start <= 0) winner = min(nv - 1, -start);
  if (winner != i) return;
  const int page = ClampPage(a.table[int64_t(s) * a.stride + pos / PT], g.n_pages);
  const size_t ph = size_t(page) * H + h;
  const size_t src = ((size_t(s) * a.n_new + i) * H + h) * D + d;
  const _Float16 kh = static_cast<_Float16>(LoadSrc(a.k_src, src, a.src_dtype));
  const _Float16 vh = static_cast<_Float16>(LoadSrc(a.v_src, src, a.src_dtype));
  a.k[KOffset(g, ph, d, pos % PT)] = __builtin_bit_cast(uint16_t, kh);
  a.v[VOffset(g, ph, d, pos % PT)] = __builtin_bit_cast(uint16_t, vh);
}

// Eight consecutive source elements from index i (a multiple of 8, the array 16-byte aligned), rounded to f16.
__device__ __forceinline__ uint4 Rows8(const void* p, size_t i, int dt) {
  if (dt == YAHKV_F16) return *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p) + i);
  float x[8];
  if (dt == YAHKV_F32) {
    const float4 lo = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i);
    const float4 hi = *reinterpret_cast<const float4*>(static_cast<const float*>(p) + i + 4);
    x[0] = lo.x, x[1] = lo.y, x[2] = lo.z, x[3] = lo.w, x[4] = hi.x, x[5] = hi.y, x[6] = hi.z, x[7] = hi.w;
  } else {
    const uint4 w = *reinterpret_cast<const uint4*>(static_cast<const uint16_t*>(p) + i);
    const uint32_t u[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) x[e] = WidenBf16(static_cast<uint16_t>(u[e / 2] >> (16 * (e % 2))));
  }
  uint32_t o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e)
    o[e] = uint32_t(__builtin_bit_cast(uint16_t, static_cast<_Float16>(x[2 * e]))) |
           uint32_t(__builtin_bit_cast(uint16_t, static_cast<_Float16>(x[2 * e + 1]))) << 16;
  return uint4{o[0], o[1], o[2], o[3]};
}

// The same append for chunks: a workgroup takes one kv head of one aligned run of T = min(PT, 32) positions (one run
// of the V^T layout), reads the tokens' rows with 16-byte loads, turns them round in LDS and writes K as 1 KB pieces
// and the V^T run as one 16 KB piece. Which token of the chunk a slot takes (clamped positions: the last one wins)
// is decided per slot, with the rule of AppendF16.
template <int T>
__global__ __launch_bounds__(256) void AppendF16Runs(const F16Args a) {
  const Geom g = a.g;
  const int H = g.n_kv, PT = g.pt, D = g.hd, C = D / 8;
  const int h = blockIdx.y, s = blockIdx.z, tid = threadIdx.x;
  const int nv = a.n_valid != nullptr ? min(max(a.n_valid[s], 0), a.n_new) : a.n_new;
  if (nv <= 0) return;
  const int64_t start = a.start_pos[s], last_pos = int64_t(a.stride) * PT - 1;
  const int64_t lo = min(max(start, int64_t(0)), last_pos), hi = min(max(start + nv - 1, int64_t(0)), last_pos);
  const int64_t p0 = (lo / T + blockIdx.x) * T;
  if (p0 > hi) return;
  constexpr int kRow = 256 + 8;  // f16 elements per token in LDS (head_dim <= 256), padded against bank conflicts
  __shared__ __align__(16) uint16_t lk[T][kRow];
  __shared__ __align__(16) uint16_t lv[T][kRow];
  __shared__ int lsrc[T];
  if (tid < T) {
    const int64_t p = p0 + tid;
    int64_t src = p - start;
    if (p == last_pos && start + nv - 1 >= last_pos) src = nv - 1;
    if (p == 0 && start <= 0) src = min(int64_t(nv - 1), -start);
    lsrc[tid] = src >= 0 && src < nv ? static_cast<int>(src) : -1;
  }
  __syncthreads();
  for (int e = tid; e < T * C; e += 256) {
    const int t = e / C, c = e % C, src = lsrc[t];
    if (src < 0) continue;
    const size_t at = ((size_t(s) * a.n_new + src) * H + h) * D + 8 * c;
    *reinterpret_cast<uint4*>(&lk[t][8 * c]) = Rows8(a.k_src, at, a.src_dtype);
    *reinterpret_cast<uint4*>(&lv[t][8 * c]) = Rows8(a.v_src, at, a.src_dtype);
  }
  __syncthreads();
  const int page = ClampPage(a.table[int64_t(s) * a.stride + p0 / PT], g.n_pages);
  const size_t ph = size_t(page) * H + h;
  const int t0 = static_cast<int>(p0 % PT);
  for (int e = tid; e < T * C; e += 256) {  // K: 16 dims of T tokens are 32 T bytes in a row
    const int g16 = e / (2 * T), t = e / 2 % T, hf = e % 2;
    if (lsrc[t] < 0) continue;
    *reinterpret_cast<uint4*>(a.k + KOffset(g, ph, 16 * g16 + 8 * hf, t0 + t)) =
        *reinterpret_cast<const uint4*>(&lk[t][16 * g16 + 8 * hf]);
  }
  for (int e = tid; e < D * (T / 8); e += 256) {  // V^T: T tokens of a dim in a row, the dims one after the other
    const int d = e / (T / 8), j = e % (T / 8);
    uint16_t w[8];
    bool all = true;
#pragma unroll
    for (int i = 0; i < 8; ++i) w[i] = lv[8 * j + i][d], all = all && lsrc[8 * j + i] >= 0;
    uint16_t* dst = a.v + VOffset(g, ph, d, t0 + 8 * j);
    if (all) {
      *reinterpret_cast<uint4*>(dst) =
          uint4{uint32_t(w[0]) | uint32_t(w[1]) << 16, uint32_t(w[2]) | uint32_t(w[3]) << 16,
                uint32_t(w[4]) | uint32_t(w[5]) << 16, uint32_t(w[6]) | uint32_t(w[7]) << 16};
    } else {
#pragma unroll
      for (int i = 0; i < 8; ++i)
        if (lsrc[8 * j + i] >= 0) dst[i] = w[i];
    }
  }
}

__device__ __forceinline__ float HalfMax(float v) {  // over the 32 lanes of a wave half
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float HalfSum(float v) {
#pragma unroll
  for (int o = 16; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
// Eight consecutive query elements as f16, one 16- or 32-byte read (LoadQ8: bf16 and f16 sources convert exactly in the
// normal f16 range, finite values beyond it saturate). Element by element, with the type looked at for each, the
// eight loads went out one after the other.
__device__ __forceinline__ h8v Query8(const void* q, size_t i, int dt) { return LoadQ8(q, i, dt); }

// One workgroup per (stretch of keys, kv head, sequence); its four waves take the stretch's 32-key tiles in turn, each
// with its own online softmax, and merge through LDS into one partial (m, l, acc) per query head (gen_decode_attn.py:
// 97-335 leaves one per page). Score layout: lane = key (mod 32), registers r < 4 = heads 4 * (lane / 32) + r.
// P.V layout: lane = dim (mod 16), 8 keys per lane group; P rows are read back so that a lane's output rows are the
// heads whose running maximum it holds (lanes 0-15: heads 0-3, lanes 32-47: heads 4-7).
template <int D, int PT>
__global__ __launch_bounds__(64 * kWaves) void PartF16(const F16Args a) {
  constexpr int NG = D / 16;
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv;
  const int h = blockIdx.y, s = blockIdx.z, tid = threadIdx.x;
  // Workgroups go to the eight XCDs in turn and the number of stretches is a multiple of eight for long contexts, so
  // stretch j of every sequence would run on XCD j % 8 and the short sequences, which have only the first few, would
  // all load the same XCDs: every (sequence, head) starts its stretches one XCD further on.
  const int split = static_cast<int>((blockIdx.x + unsigned(s) * gridDim.y + h) % gridDim.x);
  const int wave = __builtin_amdgcn_readfirstlane(tid / 64), lane = tid % 64;
  const int n32 = lane % 32, half = lane / 32, n16 = lane % 16, kg = lane / 16;
  const int len = min(max(a.seq_len[s], 0), a.max_len);
  const int k_begin = split * a.keys_per_split, k_end = min(len, k_begin + a.keys_per_split);
  const size_t part = ((size_t(s) * H + h) * a.n_splits + split) * G;
  if (k_begin >= k_end) {  // nothing of this sequence here: l = 0, which the reduce skips
    if (tid < G) a.ml[(part + tid) * 2] = kLowest, a.ml[(part + tid) * 2 + 1] = 0.0f;
    return;
  }
  __shared__ __align__(16) _Float16 lq[NG][2][8][8];  // [16-dim group][k half][head row]: 8 dims
  __shared__ __align__(16) _Float16 lp[kWaves][kMaxHeads][kTileKeys];
  __shared__ float lml[kWaves][kMaxHeads][2];
  __shared__ __align__(16) float slab[kWaves][kMaxHeads][D];
  for (int e = tid; e < NG * 16; e += 64 * kWaves) {
    const int g16 = e / 16, hf = (e / 8) % 2, rw = e % 8;
    h8v v = {0, 0, 0, 0, 0, 0, 0, 0};
    if (rw < G) v = Query8(a.q, (size_t(s) * g.n_q + size_t(h) * G + rw) * D + 16 * g16 + 8 * hf, a.q_dtype);
    *reinterpret_cast<h8v*>(&lq[g16][hf][rw][0]) = v;
  }
  __syncthreads();
  const int32_t* row = a.table + int64_t(s) * a.stride;
  const float qk = a.scale * kLog2e;  // softmax in base 2
  const int prow = n16 < 4 ? n16 : (n16 >= 8 && n16 < 12 ? n16 - 4 : 0);
  float m[4], lsum[4];
  f4v o[NG];
#pragma unroll
  for (int r = 0; r < 4; ++r) m[r] = kLowest, lsum[r] = 0.0f;
#pragma unroll
  for (int nt = 0; nt < NG; ++nt) o[nt] = f4v{0.0f, 0.0f, 0.0f, 0.0f};
  const int n_tiles = (k_end - k_begin + kTileKeys - 1) / kTileKeys;
  for (int t = wave; t < n_tiles; t += kWaves) {
    const int key0 = k_begin + kTileKeys * t;
    h8v kb[NG], vb[NG];
    {  // K: this lane's key, 8 dims of every 16-dim group
      const int key = key0 + n32;
      const int page = ClampPage(row[min(key / PT, a.stride - 1)], g.n_pages);
      const uint16_t* kp = a.k + (size_t(page) * H + h) * (size_t(D) * PT) + (key % PT) * 16 + 8 * half;
#pragma unroll
      for (int g16 = 0; g16 < NG; ++g16) kb[g16] = StreamLoad(reinterpret_cast<const h8v*>(kp + g16 * PT * 16));
    }
    {  // V^T: this lane's dim of every 16-dim tile, 8 keys (they lie in one page: pages hold multiples of 16 tokens)
      const int key = key0 + 8 * kg;
      const int page = ClampPage(row[min(key / PT, a.stride - 1)], g.n_pages);
      constexpr int RUN = PT < 32 ? PT : 32;
      const uint16_t* vp =
          a.v + (size_t(page) * H + h) * (size_t(D) * PT) + (key % PT / RUN * D + n16) * RUN + key % RUN;
#pragma unroll
      for (int nt = 0; nt < NG; ++nt) vb[nt] = StreamLoad(reinterpret_cast<const h8v*>(vp + 16 * nt * RUN));
    }
    f16v c = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int g16 = 0; g16 < NG; ++g16) {
      const h8v qa = *reinterpret_cast<const h8v*>(&lq[g16][half][n32 % 8][0]);
      c = __builtin_amdgcn_mfma_f32_32x32x16_f16(qa, kb[g16], c, 0, 0, 0);
    }
    // ---- online softmax (base 2); keys at or past the end are masked by select
    const bool valid = key0 + n32 < k_end;
    float alpha[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float sc = valid ? c[r] * qk : kLowest;
      const float mn = fmaxf(m[r], HalfMax(sc));  // finite: the tile has at least one key
      alpha[r] = __builtin_amdgcn_exp2f(m[r] - mn);
      m[r] = mn;
      const float p = __builtin_amdgcn_exp2f(sc - mn);
      lsum[r] = __builtin_fmaf(lsum[r], alpha[r], p);  // per lane; summed over the lanes at the end
      lp[wave][4 * half + r][n32] = static_cast<_Float16>(p);
    }
#pragma unroll
    for (int nt = 0; nt < NG; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[nt][r] *= alpha[r];
    if (key0 + kTileKeys > k_end) {  // the stretch's last tile: what lies past the end may be anything, also NaN
#pragma unroll
      for (int nt = 0; nt < NG; ++nt)
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (key0 + 8 * kg + j >= k_end) vb[nt][j] = static_cast<_Float16>(0.0f);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const h8v pa = *reinterpret_cast<const h8v*>(&lp[wave][prow][8 * kg]);
#pragma unroll
    for (int nt = 0; nt < NG; ++nt) o[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(pa, vb[nt], o[nt], 0, 0, 0);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();  // lp is rewritten by the next tile
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
  // ---- the four waves' partials become one: weights 2^(m_w - M), summed in wave order
  if (wave < n_tiles) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float l = HalfSum(lsum[r]);
      const int head = 4 * half + r;
      if (n32 == 0 && head < G) lml[wave][head][0] = m[r], lml[wave][head][1] = l;
    }
    if (kg == 0 || kg == 2) {
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int head = 2 * kg + r;
        if (head < G) {
#pragma unroll
          for (int nt = 0; nt < NG; ++nt) slab[wave][head][16 * nt + n16] = o[nt][r];
        }
      }
    }
  } else if (lane < G) {
    lml[wave][lane][0] = kLowest, lml[wave][lane][1] = 0.0f;
  }
  __syncthreads();
  for (int e = tid; e < G * D; e += 64 * kWaves) {
    const int head = e / D, dim = e % D;
    float mm = kLowest;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) mm = lml[w][head][1] > 0.0f ? fmaxf(mm, lml[w][head][0]) : mm;
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float v = slab[w][head][dim];  // (not written by a wave without tiles: not used then)
      if (lml[w][head][1] > 0.0f) sum = __builtin_fmaf(__builtin_amdgcn_exp2f(lml[w][head][0] - mm), v, sum);
    }
    a.acc[(part + head) * D + dim] = sum;
  }
  if (tid < G) {
    float mm = kLowest, l = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) mm = lml[w][tid][1] > 0.0f ? fmaxf(mm, lml[w][tid][0]) : mm;
#pragma unroll
    for (int w = 0; w < kWaves; ++w)
      if (lml[w][tid][1] > 0.0f) l = __builtin_fmaf(__builtin_amdgcn_exp2f(lml[w][tid][0] - mm), lml[w][tid][1], l);
    a.ml[(part + tid) * 2] = mm * kLn2, a.ml[(part + tid) * 2 + 1] = l;
  }
}

// One workgroup per (query head, sequence): the stretches' partials merged with the weights e^(m_p - M), normalized,
// and the optional sigmoid gate (gen_decode_attn.py:338-411). The weights are computed once, by one thread per
// stretch, and kept in LDS; then one thread per dim sums the stretches, eight loads in flight and no branch between
// them (a stretch without keys has weight 0 and its row, which nobody wrote, is read but not used). A sequence of
// length 0 gives 0.
constexpr int kMaxSplits = 1024;
__global__ __launch_bounds__(256) void ReduceF16(const F16Args a) {
  const Geom g = a.g;
  const int G = g.group(), H = g.n_kv, D = g.hd;
  const int hq = blockIdx.x, s = blockIdx.y, t = threadIdx.x;
  const int h = hq / G, gi = hq % G;
  const size_t p0 = (size_t(s) * H + h) * a.n_splits;
  __shared__ float w[kMaxSplits];
  __shared__ float red[4];
  float mx = kLowest;
  for (int p = t; p < a.n_splits; p += 256) {
    const float* e = a.ml + ((p0 + p) * G + gi) * 2;
    if (e[1] > 0.0f) mx = fmaxf(mx, e[0]);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  if (t % 64 == 0) red[t / 64] = mx;
  __syncthreads();
  const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  float lpart = 0.0f;
  for (int p = t; p < a.n_splits; p += 256) {
    const float* e = a.ml + ((p0 + p) * G + gi) * 2;
    const float wp = e[1] > 0.0f ? __expf(e[0] - M) : 0.0f;
    w[p] = wp;
    lpart = e[1] > 0.0f ? __builtin_fmaf(wp, e[1], lpart) : lpart;
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) lpart += __shfl_xor(lpart, o, 64);
  __syncthreads();  // red has been read, w is written
  if (t % 64 == 0) red[t / 64] = lpart;
  __syncthreads();
  const float L = (red[0] + red[1]) + (red[2] + red[3]);
  if (t >= D) return;
  float v = 0.0f;
  const float* rows = a.acc + (p0 * G + gi) * D + t;
  const size_t step = size_t(G) * D;
  int p = 0;
  for (; p + 8 <= a.n_splits; p += 8) {
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) x[j] = rows[(p + j) * step];
#pragma unroll
    for (int j = 0; j < 8; ++j) v = w[p + j] > 0.0f ? __builtin_fmaf(w[p + j], x[j], v) : v;
  }
  for (; p < a.n_splits; ++p) {
    const float x = rows[p * step];
    v = w[p] > 0.0f ? __builtin_fmaf(w[p], x, v) : v;
  }
  const size_t o = (size_t(s) * g.n_q + hq) * D + t;
  v = L > 0.0f ? v / L : 0.0f;
  if (a.gate != nullptr) v *= 1.0f / (1.0f + __expf(-a.gate[o]));
  a.out[o] = v;
}

// ---- host side ----------------------------------------------------------------------------------------------------------

int CheckF16Geometry(const yahkv_geometry* g) {
  if (g == nullptr) return YAHKV_ERR_ARG;
  if (g->format != YAHKV_KV_F16) return YAHKV_ERR_SHAPE;
  yahkv_geometry q = *g;
  q.format = YAHKV_Q8_0;  // the same limits on heads, head_dim, page size and pool as the quantized formats
  return CheckGeometry(&q);
}

// Geometry, then the two pools: not null, 16-byte aligned, each at least as long as the geometry needs.
int CheckF16Pools(const yahkv_geometry* g, const yahkv_f16_pools* pools) {
  if (const int st = CheckF16Geometry(g)) return st;
  if (pools == nullptr || pools->k == nullptr || pools->v == nullptr) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(pools->k) | reinterpret_cast<uintptr_t>(pools->v)) & 15) return YAHKV_ERR_ARG;
  const size_t need = size_t(g->n_pages) * g->n_kv_heads * g->head_dim * g->page_tokens * 2;
  if (pools->k_bytes < need || pools->v_bytes < need) return YAHKV_ERR_ARG;
  return YAHKV_OK;
}

struct Split {
  int32_t n_splits, keys_per_split;
  size_t off_acc, bytes;
};
// Stretches of every sequence: enough workgroups for a few per CU, a stretch a multiple of the four waves' tiles.
Split MakeSplit(const Geom& g, int32_t n_seqs, int32_t max_len, const yahkv_decode_options* opt) {
  Split sp;
  const int64_t unit = int64_t(kTileKeys) * kWaves;
  const int64_t pairs = int64_t(n_seqs) * g.n_kv;
  // workgroups in all: about sixteen per CU unless the caller's options say otherwise
  const int64_t target = opt != nullptr && opt->n_chunks > 0 ? opt->n_chunks : 4096;
  int64_t want = std::max<int64_t>(1, (target + pairs - 1) / pairs);
  want = std::min<int64_t>(std::min<int64_t>(want, kMaxSplits), (int64_t(max_len) + unit - 1) / unit);
  const int64_t keys = ((int64_t(max_len) + want - 1) / want + unit - 1) / unit * unit;
  sp.keys_per_split = static_cast<int32_t>(keys);
  sp.n_splits = static_cast<int32_t>((int64_t(max_len) + keys - 1) / keys);
  const size_t parts = size_t(n_seqs) * g.n_kv * sp.n_splits * g.group();
  sp.off_acc = (parts * 2 * sizeof(float) + 255) & ~size_t(255);
  sp.bytes = sp.off_acc + parts * g.hd * sizeof(float);
  return sp;
}

}  // namespace
}  // namespace yahkv

using namespace yahkv;

extern "C" size_t yahkv_f16_pool_bytes(const yahkv_geometry* g) {
  if (CheckF16Geometry(g)) return 0;
  return size_t(g->n_pages) * g->n_kv_heads * g->head_dim * g->page_tokens * 2;
}

extern "C" int yahkv_f16_append(const yahkv_geometry* g, const yahkv_f16_pools* pools, const int32_t* page_table,
                                int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid,
                                int32_t n_seqs, int32_t n_new, const void* k_src, const void* v_src,
                                int32_t src_dtype, void* stream) {
  if (const int st = CheckF16Pools(g, pools)) return st;
  if (page_table == nullptr || start_pos == nullptr || k_src == nullptr || v_src == nullptr) return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || n_new <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (src_dtype != YAHKV_F32 && src_dtype != YAHKV_F16 && src_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if (n_seqs > 65535) return YAHKV_ERR_SHAPE;  // the grid's z extent
  F16Args a{};
  a.g = MakeGeom(*g), a.k = static_cast<uint16_t*>(pools->k), a.v = static_cast<uint16_t*>(pools->v);
  a.table = page_table, a.stride = page_table_stride, a.start_pos = start_pos, a.n_valid = n_valid;
  a.n_seqs = n_seqs, a.n_new = n_new, a.k_src = k_src, a.v_src = v_src, a.src_dtype = src_dtype;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const bool aligned = ((reinterpret_cast<uintptr_t>(k_src) | reinterpret_cast<uintptr_t>(v_src)) & 15) == 0;
  if (n_new >= kRunAppendMinTokens && aligned) {  // chunks: a workgroup per run of positions
    const int T = std::min(a.g.pt, 32);
    const dim3 grid(static_cast<unsigned>((n_new + T - 2) / T + 1), static_cast<unsigned>(a.g.n_kv),
                    static_cast<unsigned>(n_seqs));
    if (T == 32) hipLaunchKernelGGL(AppendF16Runs<32>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(AppendF16Runs<16>, grid, dim3(256), 0, st, a);
    return LaunchStatus();
  }
  const dim3 grid(static_cast<unsigned>(n_new), static_cast<unsigned>(a.g.n_kv), static_cast<unsigned>(n_seqs));
  hipLaunchKernelGGL(AppendF16, grid, dim3(256), 0, st, a);
  return LaunchStatus();
}

extern "C" size_t yahkv_f16_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                                   const yahkv_decode_options* opt) {
  if (CheckF16Geometry(g) || n_seqs <= 0 || max_seq_len <= 0) return 0;
  return MakeSplit(MakeGeom(*g), n_seqs, max_seq_len, opt).bytes;
}

extern "C" int yahkv_f16_decode_attend(const yahkv_geometry* g, const yahkv_f16_pools* pools,
                                       const int32_t* page_table, int32_t page_table_stride, const int32_t* seq_len,
                                       int32_t n_seqs, int32_t max_seq_len, const void* q, int32_t q_dtype,
                                       float softmax_scale, const float* gate, float* out, void* workspace,
                                       size_t workspace_bytes, const yahkv_decode_options* opt, void* stream) {
  if (const int st = CheckF16Pools(g, pools)) return st;
  if (page_table == nullptr || seq_len == nullptr || q == nullptr || out == nullptr || workspace == nullptr)
    return YAHKV_ERR_ARG;
  if (n_seqs <= 0 || max_seq_len <= 0 || page_table_stride <= 0) return YAHKV_ERR_ARG;
  if (q_dtype != YAHKV_F32 && q_dtype != YAHKV_F16 && q_dtype != YAHKV_BF16) return YAHKV_ERR_ARG;
  if ((reinterpret_cast<uintptr_t>(workspace) | reinterpret_cast<uintptr_t>(q)) & 15) return YAHKV_ERR_ARG;
  if (n_seqs > 65535) return YAHKV_ERR_SHAPE;
  F16Args a{};
  a.g = MakeGeom(*g);
  const Split sp = MakeSplit(a.g, n_seqs, max_seq_len, opt);
  if (workspace_bytes < sp.bytes) return YAHKV_ERR_WORKSPACE;
  a.k = static_cast<uint16_t*>(pools->k), a.v = static_cast<uint16_t*>(pools->v);
  a.table = page_table, a.stride = page_table_stride, a.seq_len = seq_len, a.n_seqs = n_seqs;
  // lengths read on the device are clamped to the host's bound and to the table's extent
  a.max_len = static_cast<int32_t>(std::min<int64_t>(max_seq_len, int64_t(page_table_stride) * a.g.pt));
  a.q = q, a.q_dtype = q_dtype, a.scale = softmax_scale, a.gate = gate, a.out = out;
  a.ml = static_cast<float*>(workspace);
  a.acc = reinterpret_cast<float*>(static_cast<char*>(workspace) + sp.off_acc);
  a.n_splits = sp.n_splits, a.keys_per_split = sp.keys_per_split;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(sp.n_splits), static_cast<unsigned>(a.g.n_kv), static_cast<unsigned>(n_seqs));
#define YAHKV_LAUNCH_F16(DD, PP) hipLaunchKernelGGL((PartF16<DD, PP>), grid, dim3(64 * kWaves), 0, st, a)
  if (a.g.hd == 256 && a.g.pt == 64) YAHKV_LAUNCH_F16(256, 64);
  else if (a.g.hd == 256 && a.g.pt == 32) YAHKV_LAUNCH_F16(256, 32);
  else if (a.g.hd == 256) YAHKV_LAUNCH_F16(256, 16);
  else if (a.g.pt == 64) YAHKV_LAUNCH_F16(128, 64);
  else if (a.g.pt == 32) YAHKV_LAUNCH_F16(128, 32);
  else YAHKV_LAUNCH_F16(128, 16);
#undef YAHKV_LAUNCH_F16
  if (const int rc = LaunchStatus()) return rc;
  hipLaunchKernelGGL(ReduceF16, dim3(static_cast<unsigned>(a.g.n_q), static_cast<unsigned>(n_seqs)), dim3(256), 0, st,
                     a);
  return LaunchStatus();
}
