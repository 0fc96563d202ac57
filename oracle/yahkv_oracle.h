/* TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * CPU restatement of the reference's algorithm for the paged quantized KV path. Only tests, the smoke check
 * and the benchmark's CPU-baseline leg may call it, and only as the checker; the library under test never
 * links or loads it.
 *
 * Pinning status of each function (what proves the restatement is right):
 *   orc_quantize_q8_0      bit-exact against the reference's own yah::core::QuantizeQ8_0 compiled from its
 *                          source (oracle/_ref) and against committed golden vectors made with it
 *   orc_dequantize_q8_0/4_0  bit-exact against the reference's yah::core::Dequantize (oracle/_ref) + golden vectors
 *   orc_f16 / bf16 conversions  brute force over all 65536 bit patterns and directed f32 cases against numpy
 *   orc_quantize_q4_0      the reference has no q4_0 quantizer; this restates ggml's published
 *                          quantize_row_q4_0_ref (llama.cpp ggml-quants.c, the file
 *                          engine/core/gguf_quant.cpp:1 cites; not vendored, no version pinned by the
 *                          reference). Pinned by known answers worked out by hand from that rule
 *                          (tests/q4_known_answers.py: halves round up, the clip at code 15, the first of two
 *                          equal magnitudes decides the sign of the scale at every pair of positions, a
 *                          scale that is no power of two, the zero block) and by its invariants on random data
 *   orc_append / orc_gather_blocks  page scatter: gather-through-table == contiguous quantize, poison-fill
 *                          proves untouched bytes, brute force on tiny inputs
 *   orc_decode_attend      float64 closed-form softmax over dequantized K/V (what
 *                          engine/gpu/loom/tools/dattn_q_check.py:193-203 does) and special cases
 *   orc_prefill_attend     same closed form with the causal mask; chunk of 1 == decode
 *   orc_norm_rope          the reference holds no vectors for its norm + RoPE kernel; pinned by a hand-computed
 *                          known answer that tells the half-split pairing from the interleaved one, by pos = 0
 *                          (rotation is the identity), by the norms of rotated pairs, by the relative-position
 *                          property of the dot product, and against an independent float64 numpy form
 */
#ifndef YAHKV_ORACLE_H_
#define YAHKV_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct orc_geometry {
  int32_t format;      /* 8 = q8_0, 4 = q4_0 */
  int32_t n_q_heads;
  int32_t n_kv_heads;
  int32_t head_dim;
  int32_t page_tokens;
  int32_t n_pages;
} orc_geometry;

typedef struct orc_pools {
  uint8_t* kq;
  uint16_t* ks;
  uint8_t* vq;
  uint16_t* vs;
} orc_pools;

uint16_t orc_f32_to_f16(float f);
float orc_f16_to_f32(uint16_t h);
uint16_t orc_f32_to_bf16(float f);
float orc_bf16_to_f32(uint16_t h);
/* element-wise over arrays, for the brute-force tests */
void orc_f32_to_f16_n(const float* x, uint64_t n, uint16_t* y);
void orc_f16_to_f32_n(const uint16_t* x, uint64_t n, float* y);
void orc_f32_to_bf16_n(const float* x, uint64_t n, uint16_t* y);
void orc_bf16_to_f32_n(const uint16_t* x, uint64_t n, float* y);

/* n elements (a multiple of 32) to 34-byte / 18-byte ggml blocks and back. */
void orc_quantize_q8_0(const float* x, uint64_t n, uint8_t* dst);
void orc_quantize_q4_0(const float* x, uint64_t n, uint8_t* dst);
void orc_dequantize_q8_0(const uint8_t* src, uint64_t n, float* y);
void orc_dequantize_q4_0(const uint8_t* src, uint64_t n, float* y);

size_t orc_kq_bytes(const orc_geometry* g);
size_t orc_ks_bytes(const orc_geometry* g);
size_t orc_vq_bytes(const orc_geometry* g);
size_t orc_vs_bytes(const orc_geometry* g);

/* k_src / v_src: f32 [n_seqs][n_new][H][D] (f16 / bf16 sources are widened by the caller, which is exact). */
void orc_append(const orc_geometry* g, const orc_pools* pools, const int32_t* table, int32_t stride,
                const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs, int32_t n_new,
                const float* k_src, const float* v_src);
/* Per-row RMSNorm and NeoX (half-split) RoPE, in f32 in the reference's order of operations
 * (engine/gpu/loom/yah_fused_qk_rope_f32.loom:96-146): x, out [n_rows][D]; pos [n_rows]; weight [D] or NULL. */
void orc_norm_rope(const float* x, const float* weight, int32_t n_rows, int32_t head_dim, int32_t rotary_dim,
                   float theta, float eps, const int32_t* pos, float* out);
/* tokens [0, n_tokens) of one sequence as ggml blocks [n_tokens][H][NB][34|18]. */
void orc_gather_blocks(const orc_geometry* g, const orc_pools* pools, const int32_t* table_row, int32_t n_tokens,
                       uint8_t* dst_k, uint8_t* dst_v);
/* q f32 [n_seqs][n_q_heads][D]; gate f32 or NULL; out f32. */
void orc_decode_attend(const orc_geometry* g, const orc_pools* pools, const int32_t* table, int32_t stride,
                       const int32_t* seq_len, int32_t n_seqs, const float* q, float softmax_scale,
                       const float* gate, float* out);
/* q f32 [n_seqs][chunk_len][n_q_heads][D]; out f32 same shape. Exact arithmetic on the dequantized values: f64 sums,
 * one global maximum (nothing of a matrix unit's operand rounding is modelled). */
void orc_prefill_attend(const orc_geometry* g, const orc_pools* pools, const int32_t* table, int32_t stride,
                        const int32_t* prefix_len, int32_t n_seqs, int32_t chunk_len, const float* q,
                        float softmax_scale, const float* gate, float* out);
/* worker threads the attend functions use */
int32_t orc_threads(void);
/* Checks an identity a kernel may use in place of lround (gguf_quant.cpp:316): for every float r with bit pattern
 * magnitude in [first_bits, last_bits], both signs, lroundf(r) against the truncation of r + copysignf(0.5 - 2^-25, r).
 * Returns the number of values that differ. */
uint64_t orc_lround_identity_mismatches(uint32_t first_bits, uint32_t last_bits);

#ifdef __cplusplus
}
#endif
#endif
