/* TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's own KV formats, kv8a16 and kv4a16 (docs/architecture.md:214-230): K as int8
 * around a per-channel mean with one scale per (token, kv head, 128-dim half), or rotated by H256 and quantized to 16
 * levels per 32-dim group; V as uint8 (or 15 levels) per channel per 16-key tile around the tile's midrange, stored
 * transposed, the newest tile kept open in f16. Only tests, the smoke check and the
 * benchmark's checks may call it, and only as the checker; the library under test never links or loads it.
 *
 * Pinning status of each function:
 *   orc_kv8_quant_k / deq_k / quant_vtile / deq_vtile
 *       bit-exact against tests/golden/kv8a16_vectors.npz, which holds inputs and outputs of the reference's own numpy
 *       model of the format (quant_k, deq_k, quant_vtile, deq_vtile of engine/gpu/loom/tools/dattn_q_check.py:61-137;
 *       written by tests/golden/make_kv8a16_vectors.py): directed rows and tiles (dead halves, round-half-even ties,
 *       scales beyond the f16 range, constant tiles) and the checker's whole recipe (rng 5, T 1024, pos 700:
 *       every scale, every V stat, the open tile, digests of the code pools and sampled rows of them)
 *   orc_kv8_append (page scatter, open tile, tile closing on the 16th key, chunk form)
 *       the recipe's pools and its three append cases (:210-250) bit for bit; gather == contiguous, poison fill
 *   orc_kv8_dense (the dequantized model the attention is held to: every closed tile from codes, the newest from f16)
 *       digests of the recipe's Kd / Vd; attention over it against the recipe's own float64 result (rc_ref)
 *   orc_kv8_dense_f16 (the prefill's decode, one f16 fma per element, gen_attn_fa.py:4648-4861)
 *       parity unpinned at the bit level: the reference holds no vectors for yah_kdeq8 / yah_vdeq8 and its numpy
 *       model has no f16 form; pinned by the mathematics only (it is the correctly rounded f16 of the exact
 *       value f * S + C', checked against float64 and against deq_k / deq_vtile within half an f16 step)
 *   orc_kv4_hadamard256 / quant_k / deq_k / rotate_q (kv4a16's K: H256 of the head, 16 levels per 32-dim group)
 *       tests/golden/kv4a16_vectors.npz (written by tests/golden/make_kv4a16_vectors.py from the same numpy model with
 *       bits = 4 and its Hadamard matrix): bit-exact on rows built so that the rotation is exact in any order of sums
 *       (ties, dead groups, ranges that are no power of two, negative lows); on random rows and on the checker's recipe
 *       within what the rotation's rounding allows (the model rotates in float64, the kernel and this file in f32 in
 *       the generator's order: a code may move by one step where a value sits on a rounding boundary, under 0.2 % of
 *       the codes, which is what the reference's own checker accepts, dattn_q_check.py:222-225); the butterfly's sign
 *       and index order against the matrix itself
 *   orc_kv4_quant_vtile / deq_vtile (15 levels per channel and tile)
 *       bit-exact against the same file: directed tiles and the recipe's pools, stats, sampled tiles and append cases
 *   orc_kv8_append / dense / dense_f16 with k_bits or v_bits 4
 *       the recipe (as for 8 bits); the mixed formats k8v4 / k4v8 by each side equalling its own format's pools;
 *       the f16 decode of 4-bit codes parity unpinned at the bit level, as for 8 bits
 *   orc_kv8_kmean (yah_kmean's order of f32 sums, gen_kvq.py:99-163)
 *       parity unpinned at the bit level: the numpy model takes the mean as given; pinned against a float64 mean
 *       within the f32 summation bound, and by the reading of the generator's loop order
 */
#ifndef YAHKV_KV8_ORACLE_H_
#define YAHKV_KV8_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* head_dim is 256 and pages hold 256 tokens (gen_decode_attn.py:21-27); W = n_kv_heads * 256 is the row width.
 * k_bits / v_bits: 8 (kv8a16) or 4 (kv4a16), independently, as the reference's "kv q KB VB" (loom_decoder.hpp:4). */
typedef struct orc_kv8_geometry {
  int32_t n_q_heads;
  int32_t n_kv_heads;
  int32_t n_pages;
  int32_t k_bits;
  int32_t v_bits;
} orc_kv8_geometry;

/* The reference's buffers (loom_decoder.hpp:43-51), a pool of n_pages pages each:
 *   kq  u32 [n_pages * 256 rows][W / 4]       bytes u in the order (d0, d2, d1, d3) per dword
 *   ks  u32 [n_pages * 256 rows][W / 128]     f16x2 (256 s, -384 s) per 128-dim half
 *   vq  u32 [H][n_pages * 16 tiles][256][4]   dword w of a (tile, dim): keys 4 w + (0, 2, 1, 3)
 *   vs  u32 [H][n_pages * 16 tiles][256]      f16x2 (256 sf, cf - 384 sf)
 * with 4-bit K (kv4a16, gen_kvq.py:288-463): H256-rotated K - mean, 16 levels per 32-dim group
 *   kq  u32 [rows][W / 8]                     dims 2 j / 2 j + 1 of a dword's eight at bits 4 j / 16 + 4 j
 *   ks  u32 [rows][W / 32]                    f16x2 (16 s, lo - 16 s) per 32-dim group
 * with 4-bit V (gen_kvq.py gen_vqt(4)): 15 levels per channel and tile
 *   vq  u32 [H][tiles][256][2]                dword w: keys 8 w + (0, 2, 4, 6, 1, 3, 5, 7) at nibbles 0 .. 7
 *   vs  u32 [H][tiles][256]                   f16x2 (16 sf, cf - 23 sf)
 * and, one per page instead of one per decoder (the reference serves one sequence):
 *   km  f32 [n_pages][W]                      the channel means of the sequence whose first page this is
 *   vo  f16 [n_pages][W][16]                  the open tile of the sequence whose newest page this is */
typedef struct orc_kv8_pools {
  uint32_t* kq;
  uint32_t* ks;
  float* km;
  uint32_t* vq;
  uint32_t* vs;
  uint16_t* vo;
} orc_kv8_pools;

/* one K row of n_halves * 128 values (truncated to f16 first) -> n_halves * 32 dwords, n_halves f16 pairs */
void orc_kv8_quant_k(const float* k, const float* mean, int32_t n_halves, uint32_t* dw, uint16_t* sc);
void orc_kv8_deq_k(const uint32_t* dw, const uint16_t* sc, int32_t n_halves, float* out);
/* v: f16 bits [16 keys][n channels] -> dw [n][4], st [n][2]; out f32 [16][n] */
void orc_kv8_quant_vtile(const uint16_t* v, int32_t n, uint32_t* dw, uint16_t* st);
void orc_kv8_deq_vtile(const uint32_t* dw, const uint16_t* st, int32_t n, float* out);
/* kv4a16's codec (numpy model: dattn_q_check.py:77-85, 97-99, 101-137 with bits = 4). */
/* x[256] -> H256 x in place, unnormalized, in yah_kq4's order of f32 operations: stages 1, 2, 4, .. 128, the lower
 * element of a pair becomes lower + upper, the upper one lower - upper (gen_kvq.py:343-375) */
void orc_kv4_hadamard256(float* x);
/* one K row of n_heads * 256 values -> n_heads * 32 dwords, n_heads * 8 f16 pairs */
void orc_kv4_quant_k(const float* k, const float* mean, int32_t n_heads, uint32_t* dw, uint16_t* sc);
void orc_kv4_deq_k(const uint32_t* dw, const uint16_t* sc, int32_t n_heads, float* out);
/* v: f16 bits [16 keys][n channels] -> dw [n][2], st [n][2]; out f32 [16][n] */
void orc_kv4_quant_vtile(const uint16_t* v, int32_t n, uint32_t* dw, uint16_t* st);
void orc_kv4_deq_vtile(const uint32_t* dw, const uint16_t* st, int32_t n, float* out);
/* a query head's 256 values -> H256 q / 16 in f32, part_q's LDS butterfly (gen_decode_attn.py:655-683, 711-712): the
 * attention over 4-bit K takes its scores against this */
void orc_kv4_rotate_q(const float* q, float* out);

/* mean over rows [0, n_rows) of k (f32 [n_rows][W], truncated to f16 first), in yah_kmean's order of sums */
void orc_kv8_kmean(const float* k, int32_t n_rows, int32_t W, float* mean);

/* Append n_new tokens per sequence at start_pos[s] (n_valid[s] real ones, or all). k_src / v_src f32
 * [n_seqs][n_new][W]. The means are read from km[page of the sequence's position 0].
 * n_new == 1: the decoder's kappend + vappend (gen_decode_attn.py:1043-1107, 436-573): V goes to its key of the open
 *   tile, and the tile is quantized when that key is its 16th.
 * n_new >= 2: the prefill's kq8 + vq8 + vseed (gen_kvq.py:166-285, 474-730): every tile the chunk touches is
 *   quantized (keys before the chunk from the open tile, keys past the last real token repeat it), and the tile of the
 *   last real token is left in the open tile, keys past it zero. */
void orc_kv8_append(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* table, int32_t stride,
                    const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs, int32_t n_new,
                    const float* k_src, const float* v_src);
/* The first n_tokens of one sequence as the decode attention sees them (dattn_q_check.py:155-175): K - mean from
 * codes in f32; V of every tile before tile (n_tokens - 1) / 16 from codes in f32, that tile from the open f16 tile.
 * Kd, Vd f32 [n_tokens][W]. */
void orc_kv8_dense(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* table_row, int32_t n_tokens,
                   float* Kd, float* Vd);
/* The same tokens as the prefill attention sees them (yah_kdeq8 / yah_vdeq8): every element one f16 fma
 * f16(1 + u / 256) * S + C', every V tile from codes. Kd, Vd f32 [n_tokens][W] holding f16 values. */
void orc_kv8_dense_f16(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* table_row, int32_t n_tokens,
                       float* Kd, float* Vd);

#ifdef __cplusplus
}
#endif
#endif
