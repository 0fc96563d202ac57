/* yahkv: paged, block-quantized KV cache for one attention layer on one MI355X (gfx950).
 *
 * C ABI of the shared library libyahkv.so. Every entry point takes plain pointers and sizes; device
 * pointers are raw HIP device addresses, `stream` is a hipStream_t passed as void*. Entry points return
 * 0 on success or a negative yahkv_status; they never throw, never synchronize the device (the set-up call
 * yahkv_decode_calibrate aside, which waits for its own measurements) and, except for yahkv_pagepool_*, never
 * allocate.
 *
 * The entry points replace, for this path, the reference engine's kernel dispatches
 * (LoomDevice::Dispatch, engine/model/loom_runtime.hpp:372-376) issued by LoomDecoder::Step
 * (engine/model/loom_decoder.hpp:253-268) and by the prefill attention block
 * (engine/model/loom_prefill.hpp:3341-3410).
 *
 * ---------------------------------------------------------------------------------------------
 * Formats. A block is 32 consecutive head dimensions of one token of one kv head.
 *   q8_0: f16 scale d, 32 int8 codes, value = d * code   (engine/core/gguf_quant.cpp:72-75,310-320)
 *   q4_0: f16 scale d, 32 4-bit codes n in 0..15, value = d * (n - 8); byte j of the 16 code bytes holds
 *         element j in its low nibble and element j + 16 in its high nibble
 *         (engine/core/gguf_quant.cpp:48-51)
 *
 * Pools (the reference keeps codes and scales of K and V in four buffers per layer as well:
 * LoomDecoderState::kq/ks/vq/vs, engine/model/loom_decoder.hpp:43-51). With PT = page_tokens,
 * H = n_kv_heads, D = head_dim, NB = D / 32, all arrays C-order, one page after the other:
 *   q8_0  kq  int8 [n_pages][H][NB][PT][32]   codes of block (token t, block b) are 32 contiguous bytes
 *         ks  f16  [n_pages][H][PT][NB]
 *         vq  int8 [n_pages][H][D][PT]        V is stored transposed inside the page (token fastest), as the
 *                                             reference stores V^T tiles (gen_decode_attn.py:4-6)
 *         vs  f16  [n_pages][H][NB][PT]
 *   q4_0  kq  u8   [n_pages][H][NB][PT][16]   the 16 code bytes of a block, ggml nibble order
 *         ks  f16  [n_pages][H][PT][NB]
 *         vq  u8   [n_pages][H][NB][16][PT]   byte (b, j, t) = code(t, 32 b + j) | code(t, 32 b + 16 + j) << 4
 *         vs  f16  [n_pages][H][NB][PT]
 * The (scale, codes) pairs are bit-identical to the 34-byte / 18-byte ggml blocks; yahkv_gather_blocks
 * writes them back out in that array-of-blocks form.
 *
 * Page table: int32 [n_seqs][page_table_stride], entry [s][p] is the physical page that holds tokens
 * p * PT .. p * PT + PT - 1 of sequence s (engine/gpu/loom/tools/gen_kvq.py:48-71 for one sequence).
 * Lengths and positions are device-resident int32 so that steps queue without a host round trip
 * (engine/model/loom_decoder.hpp:119,131-133,239). Kernels clamp what they read from device memory
 * (positions to the table's extent, page numbers to the pool) as the reference's do
 * (gen_decode_attn.py:59-72); validate tables on the host with yahkv_validate_page_table.
 */
#ifndef YAHKV_H_
#define YAHKV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef enum yahkv_status {
  YAHKV_OK = 0,
  YAHKV_ERR_ARG = -1,        /* null pointer, non-positive count, misaligned pointer, pool shorter than the geometry needs */
  YAHKV_ERR_SHAPE = -2,      /* geometry this build has no kernel for */
  YAHKV_ERR_PAGE = -3,       /* page table entry outside the pool, or a page used twice */
  YAHKV_ERR_WORKSPACE = -4,  /* workspace smaller than yahkv_*_workspace_bytes */
  YAHKV_ERR_NOMEM = -5,      /* page pool exhausted */
  YAHKV_ERR_LAUNCH = -6      /* the HIP runtime refused the launch */
} yahkv_status;

/* "kv q KB VB" of the reference's decode.txt (loom_decoder.hpp:76-79): K and V share one format here. */
typedef enum yahkv_format {
  YAHKV_Q4_0 = 4,
  YAHKV_Q8_0 = 8,
  YAHKV_KV_F16 = 16,   /* yahkv_f16_* functions only */
  YAHKV_KV8A16 = 816,  /* the reference's own format, "kv q 8 8": yahkv_kv8_* functions only */
  YAHKV_KV4A16 = 416,  /* its 4-bit sibling, "kv q 4 4" (H256-rotated K, 16 levels; V 15 levels): yahkv_kv8_* functions */
  YAHKV_K8V4A16 = 8416, /* "kv q 8 4": K as kv8a16, V as kv4a16 */
  YAHKV_K4V8A16 = 4816  /* "kv q 4 8" */
} yahkv_format;
typedef enum yahkv_dtype { YAHKV_F32 = 0, YAHKV_F16 = 1, YAHKV_BF16 = 2 } yahkv_dtype;

typedef struct yahkv_geometry {
  int32_t format;       /* yahkv_format */
  int32_t n_q_heads;    /* a multiple of n_kv_heads; at most 8 query heads per kv head */
  int32_t n_kv_heads;
  int32_t head_dim;     /* 128 or 256 */
  int32_t page_tokens;  /* 16, 32 or 64 */
  int32_t n_pages;      /* pages in each of the four pools */
} yahkv_geometry;

/* Device addresses of one layer's pools, 16-byte aligned, and the length of each buffer in bytes, as the reference's
 * bindings carry theirs (hrx_buffer_ref_t{buffer, offset, length}, engine/model/loom_runtime.hpp:467-478). Every entry
 * point that takes pools refuses a pool shorter than yahkv_*_bytes(g) with YAHKV_ERR_ARG before it launches anything,
 * as the reference refuses an undersized binding (engine/run/hal_run.cc:110-114, loom_decoder.hpp:186-203). */
typedef struct yahkv_pools {
  void* kq;
  void* ks;
  void* vq;
  void* vs;
  size_t kq_bytes;
  size_t ks_bytes;
  size_t vq_bytes;
  size_t vs_bytes;
} yahkv_pools;

/* Library version string and the gfx target the kernels were compiled for. */
const char* yahkv_version(void);
/* Text for a yahkv_status. */
const char* yahkv_strerror(int status);
/* 0 if this build has kernels for the geometry, else YAHKV_ERR_SHAPE / YAHKV_ERR_ARG. */
int yahkv_check_geometry(const yahkv_geometry* g);

/* Pool sizes in bytes. Replace LoomDecoder::KqBytes/KsBytes/VqBytes/VsBytes (loom_decoder.hpp:151-154). */
size_t yahkv_kq_bytes(const yahkv_geometry* g);
size_t yahkv_ks_bytes(const yahkv_geometry* g);
size_t yahkv_vq_bytes(const yahkv_geometry* g);
size_t yahkv_vs_bytes(const yahkv_geometry* g);
/* KV bytes one token occupies in the pools (all kv heads, K and V, codes and scales); the figure the
 * reference's memory plan uses per layer (engine/model/memory_plan.hpp:55). */
size_t yahkv_bytes_per_token(const yahkv_geometry* g);

/* Host check of a page table before upload: every entry of the first ceil(len[s] / PT) entries of each row
 * is in [0, n_pages) and no physical page appears twice. Replaces the loop at loom_prefill.hpp:1314-1316.
 * `table` and `seq_len` are host pointers. */
int yahkv_validate_page_table(const yahkv_geometry* g, const int32_t* table, int32_t page_table_stride,
                              const int32_t* seq_len, int32_t n_seqs);

/* Append: quantize `n_new` tokens per sequence and scatter them into their pages.
 * Token i of sequence s goes to position start_pos[s] + i. k_src / v_src are [n_seqs][n_new][H][D] of
 * src_dtype (F32, F16 or BF16) on the device. n_valid (device int32 [n_seqs], or NULL for "all n_new")
 * gives the real rows of a padded chunk: rows at or past n_valid[s] are not written.
 * Replaces yah_dattn_kappend / yah_dattn_vappend (gen_decode_attn.py:1043-1107, 436-573) for n_new = 1 and
 * yah_kq8 / yah_vq8 (gen_kvq.py:166-285, 474-660) for a prefill chunk. */
int yahkv_append(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                 int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs,
                 int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype, void* stream);

/* Append fused with per-head RMSNorm and NeoX RoPE of K (and of Q on the way, if q_src is given):
 *   normed[i] = (x[i] * rsqrt(sum x^2 / D + eps)) * weight[i]          (weight NULL = ones)
 *   pair (p, p + rotary_dim / 2), p < rotary_dim / 2, is rotated by pos / theta^(2 p / rotary_dim)
 * with pos = start_pos[s] + t; dims at or past rotary_dim are only normalised. The rotated K rows are quantized
 * into their pages (never written out as f32 unless k_out is given), V rows are quantized as they are.
 *   q_src / q_out  [n_seqs][n_new][n_q_heads][D] of src_dtype / q_out_dtype, or both NULL
 *   k_out          [n_seqs][n_new][n_kv_heads][D] f32 or NULL
 * Replaces yah_fused_qk_rope (engine/gpu/loom/yah_fused_qk_rope_f32.loom:1-10,96-241) followed by the K / V cache
 * writes, and its paged batched form for prefill chunks (engine/gpu/loom/tools/emit_prefill_pp.py:31-111). */
typedef struct yahkv_rope {
  float theta;           /* rope base, e.g. 1e7 (yah_fused_qk_rope_f32.loom:33) */
  float eps;             /* RMSNorm epsilon */
  int32_t rotary_dim;    /* a multiple of 8, 8 .. head_dim */
  const float* k_weight; /* device f32 [D] or NULL */
  const float* q_weight; /* device f32 [D] or NULL */
} yahkv_rope;
int yahkv_append_rope(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                      int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs,
                      int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype, const yahkv_rope* rope,
                      const void* q_src, void* q_out, int32_t q_out_dtype, float* k_out, void* stream);

/* Tuning values of the decode attention. A NULL pointer or a zero field means the default; nothing is read from
 * the environment or from any other process-wide state. The same options must be given to every call that shares a
 * workspace (its layout depends on them). */
typedef struct yahkv_decode_options {
  int32_t n_chunks;         /* pieces the batch's keys are cut into = workgroups of the split-K kernel; 0: one per
                               compute unit (f16 pools: workgroups aimed at in all; 0: sixteen per compute unit) */
  int32_t min_chunk_tiles;  /* fewest 64-key tiles a piece gets (each piece costs a partial); 0: 16 (8 where the
                               whole-tile kernel of wg_partials runs: one tile per wave); at least 2 */
  int32_t pair_cost;        /* what a change of (sequence, kv head) costs a workgroup, in tiles; 0: 8 (none where the
                               whole-tile kernel runs); negative: none */
  int32_t reduce_split;     /* workgroups per (query head, sequence) of the merge; 0: chosen from the batch size */
  int32_t deterministic;    /* 0 or positive (the default): the waves of a workgroup take its tiles in a fixed pattern, so
                               two calls on the same bytes with the same options give the same bits (the two waves of a
                               SIMD pace each other through their priorities, which costs nothing measurable against a
                               first-come hand-out); negative: tiles go first come, first served, and results differ by
                               about 1e-4 relative from run to run (kept for measurements) */
  int32_t xcd_weight[8];    /* relative read speeds of the eight XCDs, as yahkv_decode_calibrate measures them; the
                               chunks of a group of eight are sized by them; all 0: equal shares */
  int32_t one_launch;       /* not 0: yahkv_decode_attend issues one dispatch instead of two: the workgroup that is last
                               to finish a pair's keys merges the pair's partials itself. Same results; measured slower
                               than the two dispatches on an MI355X (partials cross between XCDs through memory), so it
                               is for callers to whom the number of dispatches matters more than the time. Its arrival
                               counts live in the workspace and must start at zero: call yahkv_decode_workspace_init
                               once on a new workspace, and again when n_seqs, max_seq_len or the options change */
  int32_t wg_partials;      /* what a workgroup leaves of the last (sequence, kv head) pair it worked on: 1: one partial,
                               merged from its waves' in LDS; 2: one per wave; 3: one per workgroup, from waves that ask
                               for a whole tile at once instead of half a tile ahead of the arithmetic (q8_0, head_dim
                               256, 64-token pages and at most two tiles per wave with a workgroup on every CU; else as
                               1): with about one tile per wave there is nothing to run ahead of, and the step of one
                               32K sequence is 5 us shorter; 0: chosen from the batch's size (3 where it applies, else 1
                               when the whole batch is at most four 64-key tiles per wave, else 2) */
  int32_t cut;              /* how the work is cut among the waves: 1: by (sequence, kv head), each wave a stretch of one
                               head's tiles; 2: by (sequence, tile), the kv heads of a tile dealt to neighbouring waves
                               (kv head counts that divide 8; not with one_launch or one partial per workgroup: those
                               cut by head), which reads a page's kv heads together: 2 - 3 % faster, and the workspace
                               holds (chunks + n_seqs) * kv heads places for partials instead of chunks + n_seqs * kv
                               heads; 0: by tile where that is possible. The kv8a16 / kv4a16 functions always cut by
                               tile where the head count allows */
} yahkv_decode_options;

/* Decode attention: one query token per sequence against keys 0 .. seq_len[s] - 1.
 *   q    [n_seqs][n_q_heads][D] of q_dtype: F32 (what the reference's kernels take, gen_decode_attn.py:576-590), F16
 *        or BF16. The kernels compute with f16 queries: F32 rounds to nearest even, BF16 converts exactly in the
 *        normal f16 range, finite values beyond +-65504 saturate there, NaN and infinities give NaN
 *   gate [n_seqs][n_q_heads][D] f32 or NULL; with a gate, out = ctx * sigmoid(gate) (gen_decode_attn.py:402-407)
 *   out  [n_seqs][n_q_heads][D] f32
 * max_seq_len is a host-side upper bound of seq_len[] (it sizes the grid and the workspace); seq_len
 * values above it are clamped. A sequence of length 0 yields zeros.
 * Replaces yah_dattn_part_q + yah_dattn_reduce (gen_decode_attn.py:576-1040, 338-411). */
size_t yahkv_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                    const yahkv_decode_options* opt);
/* Prepares a workspace for opt->one_launch: zeroes the per-(sequence, kv head) arrival counts that form keeps in it
 * (every such launch leaves them at zero again, so once per workspace and shape is enough; a launch that was aborted
 * half way needs it again). A small fill kernel on `stream`; harmless, and not needed, for the two-dispatch forms.
 * No counterpart in the reference (its reduce is always a dispatch of its own, loom_decoder.hpp:268). */
int yahkv_decode_workspace_init(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                const yahkv_decode_options* opt, void* workspace, size_t workspace_bytes, void* stream);
/* The two dispatches of a decode attention on their own, as LoomDecoder::Step issues its own (loom_decoder.hpp:259-268):
 * `part` cuts the batch into equal pieces of work from the device-resident lengths (the reference needs no cut: it
 * has one sequence and launches one workgroup per page in use) and leaves partials (M, l, acc) per piece in the
 * workspace, with the prefix sums of the lengths; `reduce` merges the partials into out. Both must be given the same
 * geometry, n_seqs, max_seq_len, page_table_stride, options and workspace, in this order on one stream; the lengths
 * must not change in between. */
int yahkv_decode_part(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                      int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                      const void* q, int32_t q_dtype, float softmax_scale, void* workspace, size_t workspace_bytes,
                      const yahkv_decode_options* opt, void* stream);
int yahkv_decode_reduce(const yahkv_geometry* g, int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs,
                        int32_t max_seq_len, const float* gate, float* out, const void* workspace,
                        size_t workspace_bytes, const yahkv_decode_options* opt, void* stream);
/* part, then reduce (one dispatch that does both with opt->one_launch). out must be 16-byte aligned. */
int yahkv_decode_attend(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                        int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                        const void* q, int32_t q_dtype, float softmax_scale, const float* gate, float* out,
                        void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt, void* stream);
/* One decode step of a layer, LoomDecoder::Step's sequence kappend, vappend, part_q, reduce
 * (loom_decoder.hpp:253-268), in two dispatches: the result is that of yahkv_append(n_new = 1, start_pos =
 * seq_len - 1) followed by yahkv_decode_attend, pools and output. seq_len[s] counts the step's own token, which goes
 * to position seq_len[s] - 1 (clamped to the table like every position, and attended to exactly when the attention
 * of the two separate calls would reach it; lengths the host's validation accepts always are); a sequence with
 * seq_len[s] <= 0 gets no token and rows of zeros. k_new, v_new: [n_seqs][H][D] of new_dtype (F32, F16 or BF16), 16-byte aligned. The split-K
 * dispatch runs over the tokens the pools already hold; the merge quantizes the new token (the append kernels'
 * arithmetic, bit for bit), writes it to its slot and adds its term. opt->one_launch is refused (YAHKV_ERR_ARG). */
int yahkv_decode_step(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                      int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                      const void* k_new, const void* v_new, int32_t new_dtype, const void* q, int32_t q_dtype,
                      float softmax_scale, const float* gate, float* out, void* workspace, size_t workspace_bytes,
                      const yahkv_decode_options* opt, void* stream);
/* The second dispatch of yahkv_decode_step on its own, for callers that issue the two themselves (a timer or other
 * work between them). The first is yahkv_decode_part with the lengths BEFORE the step (every seq_len one less; a
 * device array of its own, since lengths are read on the device) and otherwise the same arguments; this call takes
 * the lengths after the step, as yahkv_decode_step does. The split form needs every seq_len[s] <= max_seq_len (the two
 * calls clamp longer ones differently, each from the lengths it is given; yahkv_decode_step itself clamps
 * consistently). */
int yahkv_decode_step_reduce(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                             int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                             const void* k_new, const void* v_new, int32_t new_dtype, const void* q, int32_t q_dtype,
                             float softmax_scale, const float* gate, float* out, void* workspace,
                             size_t workspace_bytes, const yahkv_decode_options* opt, void* stream);
/* Measures the relative read speeds of the GPU's eight XCDs on the caller's own batch and writes them to
 * opt->xcd_weight (the other fields are read): `rounds` times, the split-K kernel runs nine times on the given arguments and
 * the shares are corrected by when each XCD's workgroups finished; one more such run measures the last correction, and
 * the weights that were measured fastest are the ones left in opt (the XCDs share the memory, so a round corrects about
 * half of what it sees; two or three rounds are enough: on a ragged batch of 64 the steps timed afterwards are 0.5 %
 * shorter than after one round and no shorter after eight). A set-up call: it synchronizes the stream and overwrites
 * the workspace. No counterpart in the reference (one sequence, one workgroup per page). */
int yahkv_decode_calibrate(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                           int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                           const void* q, int32_t q_dtype, void* workspace, size_t workspace_bytes,
                           yahkv_decode_options* opt, int32_t rounds, void* stream);

/* Diagnostics, no counterpart in the reference: a one-wave kernel on `stream` that counts shader-clock cycles over
 * `ticks` (1 .. 100000) ticks of the GPU's constant 100 MHz counter and writes {cycles, ticks} as two uint64 to
 * device memory; 100 * cycles / ticks is the shader clock in MHz at that point of the stream. The instruction-bound
 * kernels (q4_0 decode, prefill) run as fast as that clock, which is unsteady for some tens of milliseconds after an
 * idle period. */
int yahkv_shader_clock_probe(void* cycles_and_ticks, int32_t ticks, void* stream);

/* yahkv_decode_attend without a workspace argument, for callers that cannot allocate device memory (code under HIP
 * graph capture, serving loops and harnesses that forbid hipMalloc). It has no counterpart in the reference. The
 * partials go to an array that is part of the library's code object: yahkv_decode_static_scratch_bytes() = 32 MiB,
 * held on every GPU the library runs on until the process ends. A batch whose yahkv_decode_workspace_bytes() exceeds
 * (default options) returns YAHKV_ERR_WORKSPACE and launches nothing (24 / 4 heads of 256 dims: 64 sequences fit, whatever their
 * lengths). The function calls no allocator; the device of `stream` must be the current device. Every call on a GPU uses
 * that GPU's one array: calls that overlap on one GPU (two streams, two threads) race; calls on one stream do not.
 * Results are those of yahkv_decode_attend. The first call on a device looks the array's address up
 * (hipGetSymbolAddress): make it before a graph capture begins. */
size_t yahkv_decode_static_scratch_bytes(void);
int yahkv_decode_attend_static(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                               int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                               const void* q, int32_t q_dtype, float softmax_scale, const float* gate, float* out,
                               void* stream);

/* Chunked-prefill attention: query t of sequence s (t < chunk_len) sees keys 0 .. prefix_len[s] + t, which
 * must already be in the pools (append the chunk first).
 *   q    [n_seqs][chunk_len][n_q_heads][D] bf16
 *   gate [n_seqs][chunk_len][n_q_heads][D] f32 or NULL
 *   out  [n_seqs][chunk_len][n_q_heads][D] of out_dtype (F32, F16 or BF16)
 * prefix_len is device int32 [n_seqs]; max_prefix_len is its host-side upper bound; softmax_scale > 0. K, V, the
 * queries and the softmax numerators enter the matrix unit as f16 (round to nearest even; finite values beyond
 * +-65504 saturate there), as in the reference's kernel (gen_attn_fa.py:1252-1595); sums are f32. The result lies
 * within 2e-3 (max |error| / max |value|) of exact arithmetic on the dequantized K / V for F32 and F16 output; BF16
 * output adds its own rounding, up to 2^-8 of an element.
 * With a workspace of yahkv_prefill_workspace_bytes() the prefix is decoded to f16 once per call and the attention
 * kernel reads the decoded tiles (the reference's yah_kdeq8 / yah_vdeq8 into a 16-bit pool followed by yah_attn_wmma,
 * gen_attn_fa.py:4648-4861, 1589-1595); q8_0 and q4_0. With workspace NULL the tiles are decoded inside the attention
 * kernel while they are staged (gen_attn_fa.py:2664-2779, vq4_unpack for the 4-bit codes): no extra memory, slower.
 * Both give the same results up to the order of f32 sums. */
size_t yahkv_prefill_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_prefix_len,
                                     int32_t chunk_len);
/* The two dispatches of the workspace path, for callers that queue them separately (as the reference does with
 * yah_kdeq8 / yah_vdeq8 and yah_attn_wmma, loom_prefill.hpp:3378-3416): decode keys 0 .. prefix_len[s] + chunk_len
 * of every sequence into f16 tiles in the workspace; then attention of the chunk's queries over those tiles. The
 * tiles stay valid for further queries of the same chunk (e.g. another slice of heads) until the pools change.
 * One sequence's tiles of one kv head must stay under 2 GiB (max_prefix_len + chunk_len up to 2^21 tokens at
 * head_dim 256, 2^22 at 128): longer ones return YAHKV_ERR_SHAPE. */
int yahkv_prefill_decode_tiles(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                               int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs,
                               int32_t max_prefix_len, int32_t chunk_len, void* workspace, size_t workspace_bytes,
                               void* stream);
int yahkv_prefill_attend_tiles(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                               int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs,
                               int32_t max_prefix_len, int32_t chunk_len, const void* q, float softmax_scale,
                               const float* gate, void* out, int32_t out_dtype, const void* workspace,
                               size_t workspace_bytes, void* stream);
/* decode_tiles + attend_tiles when workspace is not NULL, else the one-pass kernel. */
int yahkv_prefill_attend(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* page_table,
                         int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs,
                         int32_t max_prefix_len, int32_t chunk_len, const void* q, float softmax_scale,
                         const float* gate, void* out, int32_t out_dtype, void* workspace, size_t workspace_bytes,
                         void* stream);

/* Gather the blocks of tokens [0, n_tokens) of one sequence back into ggml array-of-blocks order:
 * dst_k / dst_v are device buffers [n_tokens][H][NB][34 or 18 bytes]. `table_row` is that sequence's row of
 * the device page table. Test and export helper; shows the pool bytes equal the ggml blocks. */
int yahkv_gather_blocks(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row,
                        int32_t n_tokens, void* dst_k, void* dst_v, void* stream);

/* Host page allocator with a free list. The reference has none (its table is the identity,
 * loom_decoder.hpp:175-179); sequences own pages, freed pages are handed out again, lowest id first. */
typedef struct yahkv_pagepool yahkv_pagepool;
yahkv_pagepool* yahkv_pagepool_create(int32_t n_pages);
void yahkv_pagepool_destroy(yahkv_pagepool* p);
int32_t yahkv_pagepool_free_count(const yahkv_pagepool* p);
/* Takes n pages; writes their ids to out. YAHKV_ERR_NOMEM (and takes none) if fewer than n are free. */
int yahkv_pagepool_alloc(yahkv_pagepool* p, int32_t n, int32_t* out);
/* Returns n pages. YAHKV_ERR_PAGE (and frees none) if an id is out of range or already free. */
int yahkv_pagepool_free(yahkv_pagepool* p, const int32_t* pages, int32_t n);
/* Hands out the free pages in the order of a seeded Fisher-Yates shuffle from now on (tests and benches use
 * it for a scrambled table, as gen_decode_attn's checker does, dattn_q_check.py:151). */
void yahkv_pagepool_shuffle(yahkv_pagepool* p, uint64_t seed);
/* Shared pages: every page has an owner count (1 after alloc). retain adds an owner to allocated pages (a sequence
 * forked from a shared prefix keeps the prefix's full pages); free removes one, and a page returns to the free
 * list when its last owner lets go. refcount: owners of a page, 0 = free, -1 = no such page.
 * (The reference has no allocator; its prefix reuse is the whole-state slot, loom_prefill.hpp:976-1024.) */
int yahkv_pagepool_retain(yahkv_pagepool* pool, const int32_t* pages, int32_t n);
int32_t yahkv_pagepool_refcount(const yahkv_pagepool* pool, int32_t page);
/* yahkv_validate_page_table for tables with shared pages: a page may appear in as many rows as it has owners in
 * `pool` (never twice in one row, never a free page). */
int yahkv_validate_shared_page_table(const yahkv_geometry* g, const yahkv_pagepool* pool, const int32_t* table,
                                     int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs);

/* Copy whole pages inside the pools: page src_pages[i] -> page dst_pages[i] (device int32 arrays), all four
 * pools. For a fork: the shared prefix's last, partly filled page must be private before the fork appends. */
int yahkv_copy_pages(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* src_pages,
                     const int32_t* dst_pages, int32_t n, void* stream);

/* Slots: the sequence state of one sequence, raw, as one buffer: a 64-byte header (u64 magic "YKVSLOT1", format,
 * kv heads, head_dim, page_tokens, pages, tokens, 4 buffers) followed by the sequence's pages of kq, ks, vq, vs in
 * logical order. pack gathers them through the sequence's page-table row (device int32 [n_pages]) into `slot`
 * (device, yahkv_slot_bytes); unpack scatters a slot into the pages named by a row (any free pages of pools with
 * the same geometry); check validates a header on the host and returns the page and token counts.
 * Follows the reference's slot, `{magic, T, B, chunks, nbufs}` + raw buffers, which loads only into the same set
 * (engine/model/loom_prefill.hpp:976-1024). */
size_t yahkv_slot_bytes(const yahkv_geometry* g, int32_t n_pages);
int yahkv_slot_pack(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row, int32_t n_pages,
                    int32_t n_tokens, void* slot, void* stream);
int yahkv_slot_check(const yahkv_geometry* g, const void* header, size_t slot_bytes, int32_t* n_pages,
                     int32_t* n_tokens);
int yahkv_slot_unpack(const yahkv_geometry* g, const yahkv_pools* pools, const int32_t* table_row, int32_t n_pages,
                      const void* slot, void* stream);

/* ---- unquantized f16 pools: the reference's fp16 twins of the decode path ------------------------------------------
 * yah_dattn_kvappend (engine/gpu/loom/tools/gen_decode_attn.py:30-94), yah_dattn_part (:97-335) and yah_dattn_reduce
 * (:338-411) on pools of f16 K and f16 V^T, with the page table, positions, clamping and argument meaning of the
 * quantized functions above. geometry.format must be YAHKV_KV_F16; the other limits are the same.
 * Pool layouts per page and kv head (f16 elements): K [head_dim / 16][page_tokens][16], V^T
 * [page_tokens / R][head_dim][R] in runs of R = min(page_tokens, 32) keys;
 * each pool is yahkv_f16_pool_bytes long and 16-byte aligned. 4 * n_kv_heads * head_dim bytes per token. */
typedef struct yahkv_f16_pools {
  void* k;
  void* v;
  size_t k_bytes; /* lengths of the two buffers; shorter than yahkv_f16_pool_bytes(g): YAHKV_ERR_ARG */
  size_t v_bytes;
} yahkv_f16_pools;
size_t yahkv_f16_pool_bytes(const yahkv_geometry* g);
/* K and V rows of n_new tokens per sequence (layout and arguments as yahkv_append), rounded to f16 (nearest even,
 * the reference's fptrunc, gen_decode_attn.py:79-80) and written at their page rows. */
int yahkv_f16_append(const yahkv_geometry* g, const yahkv_f16_pools* pools, const int32_t* page_table,
                     int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs,
                     int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype, void* stream);
/* Decode attention over keys 0 .. seq_len[s] - 1 (arguments as yahkv_decode_attend, q 16-byte aligned as there): two
 * dispatches, partials of fixed stretches of every sequence, then their merge with the optional sigmoid gate. Of the
 * options only n_chunks is used. */
size_t yahkv_f16_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                        const yahkv_decode_options* opt);
int yahkv_f16_decode_attend(const yahkv_geometry* g, const yahkv_f16_pools* pools, const int32_t* page_table,
                            int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                            const void* q, int32_t q_dtype, float softmax_scale, const float* gate, float* out,
                            void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt, void* stream);
/* Chunked-prefill attention over f16 pools after the chunk has been appended with yahkv_f16_append (arguments as
 * yahkv_prefill_attend; the workspace is required): the keys' f16 tiles are put together from the pools (the reference's
 * attention reads its 16-bit K / V pool directly, gen_attn_fa.py:1589-1595), then the same attention kernel runs. */
size_t yahkv_f16_prefill_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_prefix_len,
                                         int32_t chunk_len);
int yahkv_f16_prefill_attend(const yahkv_geometry* g, const yahkv_f16_pools* pools, const int32_t* page_table,
                             int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs,
                             int32_t max_prefix_len, int32_t chunk_len, const void* q, float softmax_scale,
                             const float* gate, void* out, int32_t out_dtype, void* workspace,
                             size_t workspace_bytes, void* stream);

/* ---- kv8a16: the reference's own KV format, byte for byte ------------------------------------------------------------
 * What the reference runs when decode.txt says "kv q 8 8" (docs/architecture.md:214-230, loom_decoder.hpp:64-87).
 * geometry.format must be YAHKV_KV8A16, head_dim 256 and page_tokens 256 (gen_decode_attn.py:21-27); W = n_kv_heads *
 * 256. Buffers, in the reference's own layouts (loom_decoder.hpp:43-51,151-154), rows and tiles of a pool of n_pages pages:
 *   kq     u32 [n_pages * 256][W / 4]         K codes u = rne((f16(k) - mean) / s) + 128, s = amax / 127 per (token, kv head,
 *                                             128-dim half); bytes of a dword hold dims (d0, d2, d1, d3) (gen_kvq.py:166-285);
 *                                             row of position p: table[p / 256] * 256 + p % 256 (gen_kvq.py:48-71)
 *   ks     u32 [n_pages * 256][W / 128]       f16 pairs (256 s, -384 s), index kv head * 2 + half
 *   vq     u32 [H][n_pages * 16][256][4]      V codes per channel per 16-key tile around the tile's midrange c with step
 *                                             s = range / 254, both rounded to f16 first: u = clamp(rne((v - c) / s) + 128,
 *                                             0, 255); dword w of a (tile, dim) holds keys 4 w + (0, 2, 1, 3)
 *                                             (gen_kvq.py:474-660); tile of position p: table[p / 256] * 16 + (p / 16) % 16
 *   vs     u32 [H][n_pages * 16][256]         f16 pairs (256 s, c - 384 s)
 * and, where the reference's decoder holds one of each for its single sequence (loom_decoder.hpp:43-51: km, vopen), one
 * per page:
 *   km     f32 [n_pages][W]                   the channel means of the sequence whose FIRST page this is (yah_kmean,
 *                                             gen_kvq.py:99-163); zero them for a sequence that starts with decode steps
 *   vopen  f16 [n_pages][W][16]               the open tile of the sequence whose NEWEST page this is: the keys of the
 *                                             sequence's last 16-key tile, unquantized (gen_decode_attn.py:436-573)
 * 2336 bytes per token (kq + ks + vq + vs; architecture.md:219). All buffers 16-byte aligned.
 *
 * kv4a16 (YAHKV_KV4A16, "kv q 4 4"; architecture.md:220, gen_kvq.py:288-463 and gen_vqt(4)) through the same functions:
 *   kq     u32 [n_pages * 256][W / 8]         K - mean of a kv head rotated by the orthonormal 256-point Walsh-Hadamard
 *                                             transform (f32 butterflies, stages 1 .. 128 in order, then / 16), 16 levels per
 *                                             32-dim group: u = clamp(rne((x - lo) / s), 0, 15), s = (hi - lo) / 15; dims
 *                                             2 j / 2 j + 1 of a dword's eight at bits 4 j / 16 + 4 j
 *   ks     u32 [n_pages * 256][W / 32]        f16 pairs (16 s, lo - 16 s), index kv head * 8 + group
 *   vq     u32 [H][n_pages * 16][256][2]      15 levels: u = clamp(rne((v - c) / s) + 7, 0, 14), s = range / 14; dword w
 *                                             holds keys 8 w + (0, 2, 4, 6, 1, 3, 5, 7) at nibbles 0 .. 7
 *   vs     u32 [H][n_pages * 16][256]         f16 pairs (16 s, c - 23 s)
 * 1408 bytes per token. The attention rotates the queries the same way itself (yah_qrot / part_q's butterfly,
 * gen_attn_fa.py:4541-4611, gen_decode_attn.py:655-683): callers pass plain queries. YAHKV_K8V4A16 and YAHKV_K4V8A16
 * take K from one format and V from the other, as the reference's "kv q KB VB" allows (loom_decoder.hpp:4,76-79). */
typedef struct yahkv_kv8_pools {
  void* kq;
  void* ks;
  void* km;
  void* vq;
  void* vs;
  void* vopen;
  size_t kq_bytes; /* lengths of the six buffers; shorter than yahkv_kv8_*_bytes(g): YAHKV_ERR_ARG */
  size_t ks_bytes;
  size_t km_bytes;
  size_t vq_bytes;
  size_t vs_bytes;
  size_t vopen_bytes;
} yahkv_kv8_pools;
/* Replace LoomDecoder::KqBytes/KsBytes/VqBytes/VsBytes at "kv q 8 8" (loom_decoder.hpp:151-154). */
size_t yahkv_kv8_kq_bytes(const yahkv_geometry* g);
size_t yahkv_kv8_ks_bytes(const yahkv_geometry* g);
size_t yahkv_kv8_km_bytes(const yahkv_geometry* g);
size_t yahkv_kv8_vq_bytes(const yahkv_geometry* g);
size_t yahkv_kv8_vs_bytes(const yahkv_geometry* g);
size_t yahkv_kv8_vopen_bytes(const yahkv_geometry* g);
/* Channel means of each sequence's first chunk: mean over rows 0 .. min(n_rows, max(n_valid[s], 1)) - 1 of k_src
 * ([n_seqs][n_rows][W] of src_dtype, truncated to f16 first), in yah_kmean's fixed order of f32 sums
 * (gen_kvq.py:99-163), written to km[table[s][0]]. Call it before the append of a sequence's first chunk, as the
 * reference does on chunk 0 only (loom_prefill.hpp:3343-3345). n_valid: device int32 [n_seqs] or NULL. */
int yahkv_kv8_kmean(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                    int32_t page_table_stride, const int32_t* n_valid, int32_t n_seqs, int32_t n_rows,
                    const void* k_src, int32_t src_dtype, void* stream);
/* Append n_new tokens per sequence at positions start_pos[s] + i (arguments as yahkv_append; k_src / v_src
 * [n_seqs][n_new][W]). Positions at or past page_table_stride * 256 are not written; rows at or past n_valid[s] are
 * not written either (the reference zero-fills its single sequence's padding rows, gen_kvq.py:20; here they may
 * belong to somebody else).
 * n_new == 1 replaces yah_dattn_kappend + yah_dattn_vappend (gen_decode_attn.py:1043-1107, 436-573): the K row is
 *   quantized, V goes to its key of the open tile, and the tile is quantized when that key is its 16th.
 * n_new >= 2 replaces yah_kq8 + yah_vq8 + yah_vseed (gen_kvq.py:166-285, 474-730): every 16-key tile the chunk
 *   touches is quantized (keys before the chunk come from the open tile, keys past the last real token repeat it,
 *   gen_kvq.py:484-486), and the tile of the last real token is left in the open tile, keys past it zero. The
 *   reference's chunks start on a page boundary; here any start works. */
int yahkv_kv8_append(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                     int32_t page_table_stride, const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs,
                     int32_t n_new, const void* k_src, const void* v_src, int32_t src_dtype, void* stream);
/* Decode attention (arguments as yahkv_decode_attend): keys 0 .. seq_len[s] - 1, the closed V tiles from codes, the
 * tile of key seq_len[s] - 1 from the open tile, K - mean from codes (the mean shifts every score of a row alike and
 * cancels in the softmax, architecture.md:206). Two dispatches: split-K over the closed tiles, then the merge, which
 * also takes the open tile's keys. Replaces yah_dattn_part_q + yah_dattn_reduce (gen_decode_attn.py:576-1040,
 * 338-411). Of the options, one_launch is refused. */
size_t yahkv_kv8_decode_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_seq_len,
                                        const yahkv_decode_options* opt);
int yahkv_kv8_decode_attend(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                            int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                            const void* q, int32_t q_dtype, float softmax_scale, const float* gate, float* out,
                            void* workspace, size_t workspace_bytes, const yahkv_decode_options* opt, void* stream);
/* yahkv_decode_calibrate for these formats: the XCDs' relative read speeds on the caller's own batch into
 * opt->xcd_weight (a set-up call: synchronizes the stream, overwrites the workspace). No counterpart in the reference. */
int yahkv_kv8_decode_calibrate(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                               int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                               const void* q, int32_t q_dtype, void* workspace, size_t workspace_bytes,
                               yahkv_decode_options* opt, int32_t rounds, void* stream);
/* The two dispatches of yahkv_kv8_decode_attend and yahkv_kv8_decode_step on their own, as LoomDecoder::Step issues
 * its own (loom_decoder.hpp:259-268); both take the same lengths (whether or not they count a token still to be
 * appended, the split-K dispatch covers the 16-key tiles that are closed once it is). With k_new / v_new the merge is
 * the step's (it appends that token and attends to it), with both NULL the plain one. */
int yahkv_kv8_decode_part(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                          int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                          const void* q, int32_t q_dtype, float softmax_scale, void* workspace, size_t workspace_bytes,
                          const yahkv_decode_options* opt, void* stream);
int yahkv_kv8_decode_reduce(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                            int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                            const void* k_new, const void* v_new, int32_t new_dtype, const void* q, int32_t q_dtype,
                            float softmax_scale, const float* gate, float* out, void* workspace,
                            size_t workspace_bytes, const yahkv_decode_options* opt, void* stream);
/* One decode step, LoomDecoder::Step's kappend, vappend, part_q, reduce (loom_decoder.hpp:253-268), in two dispatches
 * (arguments as yahkv_decode_step): seq_len[s] counts the step's own token, which goes to position seq_len[s] - 1.
 * The result is that of yahkv_kv8_append(n_new = 1) followed by yahkv_kv8_decode_attend, pools and output. Steps of a
 * sequence must be contiguous, as the reference demands of its quantized V (loom_decoder.hpp:233-235): the open
 * tile must hold the keys since the last 16-key boundary. seq_len[s] must not exceed max_seq_len. */
int yahkv_kv8_decode_step(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                          int32_t page_table_stride, const int32_t* seq_len, int32_t n_seqs, int32_t max_seq_len,
                          const void* k_new, const void* v_new, int32_t new_dtype, const void* q, int32_t q_dtype,
                          float softmax_scale, const float* gate, float* out, void* workspace, size_t workspace_bytes,
                          const yahkv_decode_options* opt, void* stream);
/* yahkv_copy_pages and the slots (above) for these formats: a page's share of all six buffers (its rows of kq / ks, its
 * channel means, its open tile, and per kv head its 16 tiles of vq / vs) moves together. A slot's body is a set of pools
 * of the slot's own page count with the identity page table, in the layouts above (kq, ks, km, vq, vs, vopen one after
 * the other), behind the same 64-byte header (6 buffers, head_dim 256, 256-token pages). */
int yahkv_kv8_copy_pages(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* src_pages,
                         const int32_t* dst_pages, int32_t n, void* stream);
size_t yahkv_kv8_slot_bytes(const yahkv_geometry* g, int32_t n_pages);
int yahkv_kv8_slot_pack(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* table_row, int32_t n_pages,
                        int32_t n_tokens, void* slot, void* stream);
int yahkv_kv8_slot_check(const yahkv_geometry* g, const void* header, size_t slot_bytes, int32_t* n_pages,
                         int32_t* n_tokens);
int yahkv_kv8_slot_unpack(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* table_row,
                          int32_t n_pages, const void* slot, void* stream);

/* The reference's own slot files ("YAHSLOT1": LoomPrefill::SaveState / LoadState, engine/model/loom_prefill.hpp:976-1024):
 * five u64 {magic, T, B, chunks, nbufs = 10}, then per buffer a u64 byte count and the raw bytes, in the order page
 * table, kq, ks, km, vq, vs, f16 K pool, f16 V^T pool, convolution rings, DeltaNet states (StateBuffers(), :1027-1030);
 * the KV buffers hold all full-attention layers one after the other, in the layouts above. parse validates a file held
 * in host memory (magic, counts, truncation, sizes that fit one of the four quantized formats with four kv heads, page
 * table entries in range) and reports what it holds; load_layer copies one layer's pages covering chunks * B tokens,
 * through the slot's page table, into pages[0 .. n) of the caller's pools (host int32, logical order; any free pages),
 * and the layer's channel means to km of pages[0]. The stream is synchronized before it returns. The recurrent states in
 * the file are skipped: they are not part of this library. */
typedef struct yahkv_refslot_info {
  uint64_t context;     /* T: the context the set was built for */
  uint64_t chunk;       /* B: its chunk size */
  uint64_t chunks;      /* chunks the slot covers: chunks * B tokens */
  int32_t n_pages;      /* entries of the slot's page table = 256-token pages of its pools */
  int32_t n_layers;     /* full-attention layers in the file */
  int32_t n_kv_heads;   /* 4 */
  int32_t format;       /* YAHKV_KV8A16, YAHKV_KV4A16, YAHKV_K8V4A16 or YAHKV_K4V8A16 */
  uint64_t offset[10];  /* where each buffer's bytes start in the file, and how many there are */
  uint64_t size[10];
} yahkv_refslot_info;
int yahkv_refslot_parse(const void* file, size_t file_bytes, yahkv_refslot_info* info);
int yahkv_refslot_load_layer(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const void* file, size_t file_bytes,
                             int32_t layer, const int32_t* pages, int32_t n_pages, void* stream);

/* Chunked-prefill attention over kv8a16 pools after the chunk has been appended (arguments as yahkv_prefill_attend;
 * the workspace is required): keys 0 .. prefix_len[s] + chunk_len are decoded once into f16 tiles with the
 * reference's own decode, one f16 fma f16(1 + u / 256) * S + C' per element, every V tile from codes (yah_kdeq8 /
 * yah_vdeq8, gen_attn_fa.py:4648-4861), then the attention kernel of yahkv_prefill_attend_tiles runs
 * (yah_attn_wmma, gen_attn_fa.py:1589-1595). */
size_t yahkv_kv8_prefill_workspace_bytes(const yahkv_geometry* g, int32_t n_seqs, int32_t max_prefix_len,
                                         int32_t chunk_len);
int yahkv_kv8_prefill_attend(const yahkv_geometry* g, const yahkv_kv8_pools* pools, const int32_t* page_table,
                             int32_t page_table_stride, const int32_t* prefix_len, int32_t n_seqs,
                             int32_t max_prefix_len, int32_t chunk_len, const void* q, float softmax_scale,
                             const float* gate, void* out, int32_t out_dtype, void* workspace,
                             size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* YAHKV_H_ */
