/* TEST INFRASTRUCTURE, NOT PRODUCT CODE: see yahkv_oracle.h for what may call this and for what pins each function.
 *
 * Plain C restatement of the reference's arithmetic for the paged quantized KV path:
 *   block bytes        engine/core/gguf_quant.cpp:17-24 (f16 conversions), 48-51 (q4_0), 72-75 (q8_0),
 *                      310-320 (QuantizeQ8_0)
 *   page mapping       engine/gpu/loom/tools/gen_kvq.py:48-71 (row = table[p / PT] * PT + p % PT, page clamped
 *                      into the pool by writers)
 *   decode attention   engine/gpu/loom/tools/gen_decode_attn.py:97-335 (one partial (M, l, acc) per page),
 *                      338-411 (merge of the pages, gate), masking key < pos + 1 (:145,167)
 *   prefill attention  engine/gpu/loom/tools/gen_attn_fa.py:1-21 (query start_pos + t sees keys 0..start_pos + t)
 * Build: gcc -O3 -ffp-contract=off -fopenmp (no -ffast-math: the rounding below is the contract).
 */
#include "yahkv_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

/* ---- f16 / bf16 (the reference converts through _Float16, round to nearest even: gguf_quant.cpp:17-24) ---- */

uint16_t orc_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  const uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  x &= 0x7fffffffu;
  if (x > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((x >> 13) & 0x3ffu)); /* NaN, quiet */
  if (x >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);                        /* >= 65536: inf */
  const uint32_t e = x >> 23;
  if (e >= 113) { /* normal f16, may round up into the next binade or to inf */
    uint32_t h = ((e - 112) << 10) | ((x & 0x7fffffu) >> 13);
    const uint32_t rem = x & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h;
    return (uint16_t)(sign | h);
  }
  const uint32_t shift = 126 - e; /* subnormal f16: value = mant * 2^-24 */
  if (shift > 25) return sign;
  const uint32_t mant = (x & 0x7fffffu) | 0x800000u;
  uint32_t h = mant >> shift;
  const uint32_t rem = mant & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (h & 1u))) ++h;
  return (uint16_t)(sign | h);
}

float orc_f16_to_f32(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16;
  uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu, x;
  if (e == 31) {
    x = sign | 0x7f800000u | (m << 13);
  } else if (e != 0) {
    x = sign | ((e + 112) << 23) | (m << 13);
  } else if (m == 0) {
    x = sign;
  } else { /* subnormal: normalize */
    e = 113;
    while (!(m & 0x400u)) m <<= 1, --e;
    x = sign | (e << 23) | ((m & 0x3ffu) << 13);
  }
  float f;
  memcpy(&f, &x, 4);
  return f;
}

uint16_t orc_f32_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x40u);
  x += 0x7fffu + ((x >> 16) & 1u);
  return (uint16_t)(x >> 16);
}

float orc_bf16_to_f32(uint16_t h) { /* gguf_quant.cpp:295-300 */
  const uint32_t x = (uint32_t)h << 16;
  float f;
  memcpy(&f, &x, 4);
  return f;
}

void orc_f32_to_f16_n(const float* x, uint64_t n, uint16_t* y) {
  for (uint64_t i = 0; i < n; ++i) y[i] = orc_f32_to_f16(x[i]);
}
void orc_f16_to_f32_n(const uint16_t* x, uint64_t n, float* y) {
  for (uint64_t i = 0; i < n; ++i) y[i] = orc_f16_to_f32(x[i]);
}
void orc_f32_to_bf16_n(const float* x, uint64_t n, uint16_t* y) {
  for (uint64_t i = 0; i < n; ++i) y[i] = orc_f32_to_bf16(x[i]);
}
void orc_bf16_to_f32_n(const uint16_t* x, uint64_t n, float* y) {
  for (uint64_t i = 0; i < n; ++i) y[i] = orc_bf16_to_f32(x[i]);
}

/* ---- blocks ---- */

/* gguf_quant.cpp:310-320. std::max(amax, a) keeps amax unless amax < a; lround rounds halves away from zero. */
void orc_quantize_q8_0(const float* x, uint64_t n, uint8_t* dst) {
  for (uint64_t b = 0; b < n / 32; ++b, x += 32, dst += 34) {
    float amax = 0;
    for (int i = 0; i < 32; ++i) {
      const float a = fabsf(x[i]);
      if (amax < a) amax = a;
    }
    const float d = amax / 127.0f, inv = d > 0 ? 1.0f / d : 0.0f;
    const uint16_t hd = orc_f32_to_f16(d);
    memcpy(dst, &hd, 2);
    for (int i = 0; i < 32; ++i) dst[2 + i] = (uint8_t)(int8_t)lroundf(x[i] * inv);
  }
}

/* ggml quantize_row_q4_0_ref: the element of largest magnitude (first one on ties) maps to code 0 (-8 d). */
void orc_quantize_q4_0(const float* x, uint64_t n, uint8_t* dst) {
  for (uint64_t b = 0; b < n / 32; ++b, x += 32, dst += 18) {
    float amax = 0, max = 0;
    for (int i = 0; i < 32; ++i) {
      const float v = x[i];
      if (amax < fabsf(v)) amax = fabsf(v), max = v;
    }
    const float d = max / -8.0f, id = d != 0 ? 1.0f / d : 0.0f;
    const uint16_t hd = orc_f32_to_f16(d);
    memcpy(dst, &hd, 2);
    for (int j = 0; j < 16; ++j) {
      const float x0 = x[j] * id, x1 = x[16 + j] * id;
      int q0 = (int8_t)(x0 + 8.5f), q1 = (int8_t)(x1 + 8.5f);
      if (q0 > 15) q0 = 15;
      if (q1 > 15) q1 = 15;
      dst[2 + j] = (uint8_t)(q0 | (q1 << 4));
    }
  }
}

void orc_dequantize_q8_0(const uint8_t* src, uint64_t n, float* y) { /* gguf_quant.cpp:72-75 */
  for (uint64_t b = 0; b < n / 32; ++b, src += 34, y += 32) {
    uint16_t hd;
    memcpy(&hd, src, 2);
    const float d = orc_f16_to_f32(hd);
    for (int j = 0; j < 32; ++j) y[j] = d * (float)(int8_t)src[2 + j];
  }
}

void orc_dequantize_q4_0(const uint8_t* src, uint64_t n, float* y) { /* gguf_quant.cpp:48-51 */
  for (uint64_t b = 0; b < n / 32; ++b, src += 18, y += 32) {
    uint16_t hd;
    memcpy(&hd, src, 2);
    const float d = orc_f16_to_f32(hd);
    for (int j = 0; j < 16; ++j) {
      y[j] = d * (float)((src[2 + j] & 0xF) - 8);
      y[j + 16] = d * (float)((src[2 + j] >> 4) - 8);
    }
  }
}

/* ---- pools ---- */

static size_t nb_of(const orc_geometry* g) { return (size_t)g->head_dim / 32; }
static size_t cb_of(const orc_geometry* g) { return g->format == 8 ? 32 : 16; } /* code bytes per block */

size_t orc_kq_bytes(const orc_geometry* g) {
  return (size_t)g->n_pages * g->n_kv_heads * nb_of(g) * g->page_tokens * cb_of(g);
}
size_t orc_ks_bytes(const orc_geometry* g) {
  return (size_t)g->n_pages * g->n_kv_heads * g->page_tokens * nb_of(g) * 2;
}
size_t orc_vq_bytes(const orc_geometry* g) { return orc_kq_bytes(g); }
size_t orc_vs_bytes(const orc_geometry* g) { return orc_ks_bytes(g); }

static int32_t clamp_page(const orc_geometry* g, int32_t pg) { /* gen_kvq.py:60-71: writers clamp into the pool */
  if (pg < 0) pg = 0;
  if (pg > g->n_pages - 1) pg = g->n_pages - 1;
  return pg;
}

/* One ggml block (scale + codes) into / out of slot (page, head, block, token). */
static void put_block(const orc_geometry* g, const orc_pools* p, int is_v, int32_t page, int h, int b, int t,
                      const uint8_t* blk) {
  const size_t H = g->n_kv_heads, NB = nb_of(g), PT = g->page_tokens, D = g->head_dim;
  const size_t ph = (size_t)page * H + h;
  uint16_t hd;
  memcpy(&hd, blk, 2);
  if (!is_v) {
    p->ks[(ph * PT + t) * NB + b] = hd;
    memcpy(p->kq + ((ph * NB + b) * PT + t) * cb_of(g), blk + 2, cb_of(g));
  } else {
    p->vs[(ph * NB + b) * PT + t] = hd;
    if (g->format == 8)
      for (int j = 0; j < 32; ++j) p->vq[(ph * D + 32 * b + j) * PT + t] = blk[2 + j];
    else
      for (int j = 0; j < 16; ++j) p->vq[((ph * NB + b) * 16 + j) * PT + t] = blk[2 + j];
  }
}

static void get_block(const orc_geometry* g, const orc_pools* p, int is_v, int32_t page, int h, int b, int t,
                      uint8_t* blk) {
  const size_t H = g->n_kv_heads, NB = nb_of(g), PT = g->page_tokens, D = g->head_dim;
  const size_t ph = (size_t)page * H + h;
  if (!is_v) {
    memcpy(blk, &p->ks[(ph * PT + t) * NB + b], 2);
    memcpy(blk + 2, p->kq + ((ph * NB + b) * PT + t) * cb_of(g), cb_of(g));
  } else {
    memcpy(blk, &p->vs[(ph * NB + b) * PT + t], 2);
    if (g->format == 8)
      for (int j = 0; j < 32; ++j) blk[2 + j] = p->vq[(ph * D + 32 * b + j) * PT + t];
    else
      for (int j = 0; j < 16; ++j) blk[2 + j] = p->vq[((ph * NB + b) * 16 + j) * PT + t];
  }
}

void orc_append(const orc_geometry* g, const orc_pools* pools, const int32_t* table, int32_t stride,
                const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs, int32_t n_new,
                const float* k_src, const float* v_src) {
  const int H = g->n_kv_heads, D = g->head_dim, NB = D / 32, PT = g->page_tokens;
  for (int s = 0; s < n_seqs; ++s) {
    const int rows = n_valid ? (n_valid[s] < n_new ? n_valid[s] : n_new) : n_new;
    for (int i = 0; i < rows; ++i) {
      int pos = start_pos[s] + i;
      if (pos < 0) pos = 0;
      if (pos > stride * PT - 1) pos = stride * PT - 1; /* gen_decode_attn.py:59-63: pos clamped to the table */
      const int32_t page = clamp_page(g, table[(size_t)s * stride + pos / PT]);
      for (int h = 0; h < H; ++h)
        for (int b = 0; b < NB; ++b) {
          const size_t off = (((size_t)s * n_new + i) * H + h) * D + 32 * (size_t)b;
          uint8_t blk[34];
          if (g->format == 8) orc_quantize_q8_0(k_src + off, 32, blk); else orc_quantize_q4_0(k_src + off, 32, blk);
          put_block(g, pools, 0, page, h, b, pos % PT, blk);
          if (g->format == 8) orc_quantize_q8_0(v_src + off, 32, blk); else orc_quantize_q4_0(v_src + off, 32, blk);
          put_block(g, pools, 1, page, h, b, pos % PT, blk);
        }
    }
  }
}

void orc_gather_blocks(const orc_geometry* g, const orc_pools* pools, const int32_t* table_row, int32_t n_tokens,
                       uint8_t* dst_k, uint8_t* dst_v) {
  const int H = g->n_kv_heads, NB = g->head_dim / 32, PT = g->page_tokens;
  const size_t bb = 2 + cb_of(g);
  for (int p = 0; p < n_tokens; ++p) {
    const int32_t page = clamp_page(g, table_row[p / PT]);
    for (int h = 0; h < H; ++h)
      for (int b = 0; b < NB; ++b) {
        const size_t o = (((size_t)p * H + h) * NB + b) * bb;
        get_block(g, pools, 0, page, h, b, p % PT, dst_k + o);
        get_block(g, pools, 1, page, h, b, p % PT, dst_v + o);
      }
  }
}

/* Tokens [0, n) of page `page`, kv head h, to f32 [n][D]. */
static void deq_page(const orc_geometry* g, const orc_pools* p, int is_v, int32_t page, int h, int n, float* y) {
  const int D = g->head_dim, NB = D / 32;
  uint8_t blk[34];
  for (int t = 0; t < n; ++t)
    for (int b = 0; b < NB; ++b) {
      get_block(g, p, is_v, page, h, b, t, blk);
      if (g->format == 8) orc_dequantize_q8_0(blk, 32, y + (size_t)t * D + 32 * b);
      else orc_dequantize_q4_0(blk, 32, y + (size_t)t * D + 32 * b);
    }
}

int32_t orc_threads(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}

/* gen_decode_attn.py: part (one (M, l, acc) per page and head) then reduce. All arithmetic f32. */
void orc_decode_attend(const orc_geometry* g, const orc_pools* pools, const int32_t* table, int32_t stride,
                       const int32_t* seq_len, int32_t n_seqs, const float* q, float softmax_scale,
                       const float* gate, float* out) {
  const int H = g->n_kv_heads, NQ = g->n_q_heads, G = NQ / H, D = g->head_dim, PT = g->page_tokens;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < n_seqs; ++s)
    for (int h = 0; h < H; ++h) {
      int len = seq_len[s];
      if (len > stride * PT) len = stride * PT;
      float* o = out + ((size_t)s * NQ + (size_t)h * G) * D;
      if (len <= 0) {
        memset(o, 0, sizeof(float) * (size_t)G * D);
        continue;
      }
      const int np = (len + PT - 1) / PT;
      float* kd = (float*)malloc(sizeof(float) * (size_t)PT * D * 2);
      float* vd = kd + (size_t)PT * D;
      float* acc = (float*)calloc((size_t)np * G * D, sizeof(float));
      float* ml = (float*)malloc(sizeof(float) * (size_t)np * G * 2);
      float* sc = (float*)malloc(sizeof(float) * PT);
      for (int p = 0; p < np; ++p) {
        const int n = len - p * PT < PT ? len - p * PT : PT; /* keys past len are masked (key < pos + 1) */
        const int32_t page = clamp_page(g, table[(size_t)s * stride + p]);
        deq_page(g, pools, 0, page, h, n, kd);
        deq_page(g, pools, 1, page, h, n, vd);
        for (int gi = 0; gi < G; ++gi) {
          const float* qh = q + ((size_t)s * NQ + (size_t)h * G + gi) * D;
          float M = -3.4028234663852886e+38f;
          for (int t = 0; t < n; ++t) {
            float dot = 0;
            for (int d = 0; d < D; ++d) dot += qh[d] * kd[(size_t)t * D + d];
            sc[t] = dot * softmax_scale;
            if (sc[t] > M) M = sc[t];
          }
          float l = 0;
          float* a = acc + ((size_t)p * G + gi) * D;
          for (int t = 0; t < n; ++t) {
            const float e = expf(sc[t] - M);
            l += e;
            for (int d = 0; d < D; ++d) a[d] += e * vd[(size_t)t * D + d];
          }
          ml[((size_t)p * G + gi) * 2] = M;
          ml[((size_t)p * G + gi) * 2 + 1] = l;
        }
      }
      for (int gi = 0; gi < G; ++gi) { /* reduce: gen_decode_attn.py:373-407 */
        float M = -3.4028234663852886e+38f;
        for (int p = 0; p < np; ++p) M = fmaxf(M, ml[((size_t)p * G + gi) * 2]);
        for (int d = 0; d < D; ++d) o[(size_t)gi * D + d] = 0;
        float L = 0;
        for (int p = 0; p < np; ++p) {
          const float w = expf(ml[((size_t)p * G + gi) * 2] - M);
          L += w * ml[((size_t)p * G + gi) * 2 + 1];
          for (int d = 0; d < D; ++d) o[(size_t)gi * D + d] += w * acc[((size_t)p * G + gi) * D + d];
        }
        const float inv = 1.0f / L;
        for (int d = 0; d < D; ++d) {
          float v = o[(size_t)gi * D + d] * inv;
          if (gate) v *= 1.0f / (1.0f + expf(-gate[((size_t)s * NQ + (size_t)h * G + gi) * D + d]));
          o[(size_t)gi * D + d] = v;
        }
      }
      free(kd), free(acc), free(ml), free(sc);
    }
}

/* engine/gpu/loom/yah_fused_qk_rope_f32.loom:96-146 (Q branch; the K branch :147-214 is the same arithmetic):
 * sum of squares, mean + eps, rsqrt, (x * inv_rms) * weight, then pairs (p, p + half) rotated by
 * pos * (1 / powf(theta, 2 p / rotary_dim)); dims at or past rotary_dim are only normalised (:137-146). */
void orc_norm_rope(const float* x, const float* weight, int32_t n_rows, int32_t head_dim, int32_t rotary_dim,
                   float theta, float eps, const int32_t* pos, float* out) {
  const int half = rotary_dim / 2;
  for (int r = 0; r < n_rows; ++r) {
    const float* xr = x + (size_t)r * head_dim;
    float* o = out + (size_t)r * head_dim;
    float ss = 0;
    for (int i = 0; i < head_dim; ++i) ss += xr[i] * xr[i];
    const float inv = 1.0f / sqrtf(ss / (float)head_dim + eps);
    for (int i = 0; i < head_dim; ++i) o[i] = (xr[i] * inv) * (weight ? weight[i] : 1.0f);
    const float posf = (float)pos[r];
    for (int p = 0; p < half; ++p) {
      const float invfreq = powf(theta, (2.0f * (float)p) / (float)rotary_dim);
      const float angle = posf * (1.0f / invfreq);
      const float cv = cosf(angle), sv = sinf(angle);
      const float n0 = o[p], n1 = o[p + half];
      o[p] = n0 * cv - n1 * sv;
      o[p + half] = n0 * sv + n1 * cv;
    }
  }
}

void orc_prefill_attend(const orc_geometry* g, const orc_pools* pools, const int32_t* table, int32_t stride,
                        const int32_t* prefix_len, int32_t n_seqs, int32_t chunk_len, const float* q,
                        float softmax_scale, const float* gate, float* out) {
  const int H = g->n_kv_heads, NQ = g->n_q_heads, G = NQ / H, D = g->head_dim, PT = g->page_tokens;
#pragma omp parallel for collapse(2) schedule(dynamic, 1)
  for (int s = 0; s < n_seqs; ++s)
    for (int h = 0; h < H; ++h) {
      int pre = prefix_len[s];
      if (pre < 0) pre = 0;
      if (pre > stride * PT - chunk_len) pre = stride * PT - chunk_len;
      const int n = pre + chunk_len, np = (n + PT - 1) / PT;
      float* kd = (float*)malloc(sizeof(float) * (size_t)np * PT * D * 2);
      float* vd = kd + (size_t)np * PT * D;
      double* sc = (double*)malloc(sizeof(double) * (size_t)n);
      double* acc = (double*)malloc(sizeof(double) * (size_t)D);
      for (int p = 0; p < np; ++p) {
        const int nt = n - p * PT < PT ? n - p * PT : PT;
        const int32_t page = clamp_page(g, table[(size_t)s * stride + p]);
        deq_page(g, pools, 0, page, h, nt, kd + (size_t)p * PT * D);
        deq_page(g, pools, 1, page, h, nt, vd + (size_t)p * PT * D);
      }
      for (int t = 0; t < chunk_len; ++t)
        for (int gi = 0; gi < G; ++gi) {
          const size_t row = (((size_t)s * chunk_len + t) * NQ + (size_t)h * G + gi) * D;
          const int keys = pre + t + 1; /* causal: query start + t sees keys 0..start + t */
          double M = -1e300;
          for (int k = 0; k < keys; ++k) {
            double dot = 0;
            for (int d = 0; d < D; ++d) dot += (double)q[row + d] * kd[(size_t)k * D + d];
            sc[k] = dot * softmax_scale;
            if (sc[k] > M) M = sc[k];
          }
          double l = 0;
          for (int d = 0; d < D; ++d) acc[d] = 0;
          for (int k = 0; k < keys; ++k) {
            const double e = exp(sc[k] - M);
            l += e;
            for (int d = 0; d < D; ++d) acc[d] += e * vd[(size_t)k * D + d];
          }
          for (int d = 0; d < D; ++d) {
            double v = acc[d] / l;
            if (gate) v /= 1.0 + exp(-(double)gate[row + d]);
            out[row + d] = (float)v;
          }
        }
      free(kd), free(sc), free(acc);
    }
}

uint64_t orc_lround_identity_mismatches(uint32_t first_bits, uint32_t last_bits) {
  const float c = 0x1.fffffep-2f; /* the float below one half */
  uint64_t bad = 0;
#pragma omp parallel for reduction(+ : bad) schedule(static)
  for (int64_t u = first_bits; u <= (int64_t)last_bits; ++u) {
    for (uint32_t sign = 0; sign < 2; ++sign) {
      const uint32_t bits = (uint32_t)u | (sign << 31);
      float r;
      memcpy(&r, &bits, 4);
      volatile float shifted = r + copysignf(c, r); /* one rounded addition, then the conversion truncates */
      bad += lroundf(r) != (long)shifted;
    }
  }
  return bad;
}
