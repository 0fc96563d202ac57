/* TEST INFRASTRUCTURE, NOT PRODUCT CODE: see kv8_oracle.h for what may call this and for what pins each function.
 *
 * Plain C restatement of the reference's kv8a16 arithmetic:
 *   K quantizer      engine/gpu/loom/tools/gen_kvq.py:166-285 (yah_kq8), numpy model dattn_q_check.py:61-76
 *   K decode         gen_decode_attn.py:784-804 (f32), numpy model dattn_q_check.py:91-101
 *   V tile quantizer gen_kvq.py:474-660 (yah_vq8, vqt_quant, vqt_stats), numpy model dattn_q_check.py:104-127
 *   V decode         gen_decode_attn.py:969-997 (f32), numpy model dattn_q_check.py:130-143
 *   channel mean     gen_kvq.py:99-163 (yah_kmean)
 *   one-token append gen_decode_attn.py:1043-1107 (kappend), 436-573 (vappend: open tile, quantize on the 16th key)
 *   open-tile seed   gen_kvq.py:676-730 (yah_vseed)
 *   prefill decode   gen_attn_fa.py:4648-4861 (yah_kdeq8 / yah_vdeq8: one f16 fma per element)
 *   page mapping     gen_kvq.py:48-71 (row = table[p / 256] * 256 + p % 256; V tile = table[tile / 16] * 16 + tile % 16)
 * Build: gcc -O3 -ffp-contract=off (the rounding below is the contract).
 */
#include "kv8_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>

#include "yahkv_oracle.h"

static const int kPerm4[4] = {0, 2, 1, 3}; /* byte slot b of a dword holds element kPerm4[b] of its four */

static float trunc_f16(float x) { return orc_f16_to_f32(orc_f32_to_f16(x)); }

/* a double to f16 with one rounding (to nearest, ties to even); the double is an exact sum or product of f16 values */
static uint16_t f64_to_f16(double v) {
  if (v != v) return 0x7e00u;
  const uint16_t sign = signbit(v) ? 0x8000u : 0u;
  double a = fabs(v);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u); /* rounds to infinity */
  int e;
  frexp(a, &e); /* a = m * 2^e, m in [0.5, 1) */
  int ulp_exp = (e - 1) - 10;
  if (ulp_exp < -24) ulp_exp = -24;                      /* subnormal range: fixed step 2^-24 */
  const double r = ldexp(nearbyint(ldexp(a, -ulp_exp)), ulp_exp); /* nearbyint: current mode, ties to even */
  return (uint16_t)(sign | orc_f32_to_f16((float)r));   /* r is an f16 value: exact */
}

static uint32_t code_of(float r) { /* fptosi of a value that is already integral, kept to its byte */
  if (!(r == r)) return 0;
  if (r > 2147483520.0f) return 0xFFu;
  if (r < -2147483648.0f) return 0u;
  return (uint32_t)(int32_t)r & 0xFFu;
}

void orc_kv8_quant_k(const float* k, const float* mean, int32_t n_halves, uint32_t* dw, uint16_t* sc) {
  for (int hh = 0; hh < n_halves; ++hh) {
    float x[128], amax = 0.0f;
    for (int i = 0; i < 128; ++i) {
      x[i] = trunc_f16(k[hh * 128 + i]) - mean[hh * 128 + i];
      const float a = fabsf(x[i]);
      if (a > amax) amax = a;
    }
    const float s0 = amax / 127.0f;
    const float s = s0 > 0.0f ? s0 : 1.0f;
    const float inv = 1.0f / s;
    for (int j = 0; j < 32; ++j) {
      uint32_t w = 0;
      for (int b = 0; b < 4; ++b) {
        const float q = x[4 * j + kPerm4[b]] * inv;
        w |= code_of(rintf(q) + 128.0f) << (8 * b);
      }
      dw[hh * 32 + j] = w;
    }
    sc[2 * hh] = orc_f32_to_f16(s * 256.0f);
    sc[2 * hh + 1] = orc_f32_to_f16(s * -384.0f);
  }
}

void orc_kv8_deq_k(const uint32_t* dw, const uint16_t* sc, int32_t n_halves, float* out) {
  for (int hh = 0; hh < n_halves; ++hh) {
    const float d = orc_f16_to_f32(sc[2 * hh]) / 256.0f;
    for (int j = 0; j < 32; ++j)
      for (int b = 0; b < 4; ++b) {
        const float u = (float)((dw[hh * 32 + j] >> (8 * b)) & 255u);
        out[hh * 128 + 4 * j + kPerm4[b]] = (u - 128.0f) * d;
      }
  }
}

void orc_kv8_quant_vtile(const uint16_t* v, int32_t n, uint32_t* dw, uint16_t* st) {
  for (int c = 0; c < n; ++c) {
    float x[16], mx, mn;
    for (int j = 0; j < 16; ++j) x[j] = orc_f16_to_f32(v[j * n + c]);
    mx = mn = x[0];
    for (int j = 1; j < 16; ++j) mx = fmaxf(mx, x[j]), mn = fminf(mn, x[j]);
    const float cen = (mx + mn) * 0.5f;
    const float s0 = (mx - mn) / 254.0f;
    const float s = s0 > 0.0f ? s0 : 1.0f;
    const float sf = trunc_f16(s), cf = trunc_f16(cen); /* the stats are rounded to f16 before they are used */
    const float inv = 1.0f / sf;
    for (int w = 0; w < 4; ++w) {
      uint32_t word = 0;
      for (int b = 0; b < 4; ++b) {
        const float q = (x[4 * w + kPerm4[b]] - cf) * inv;
        const float r = fminf(fmaxf(rintf(q) + 128.0f, 0.0f), 255.0f); /* fmaxf(NaN, 0) = 0, as maxnumf */
        word |= code_of(r) << (8 * b);
      }
      dw[c * 4 + w] = word;
    }
    st[2 * c] = orc_f32_to_f16(sf * 256.0f);
    st[2 * c + 1] = orc_f32_to_f16(cf + sf * -384.0f); /* sf * 384 is exact: the same as the kernel's fma */
  }
}

void orc_kv8_deq_vtile(const uint32_t* dw, const uint16_t* st, int32_t n, float* out) {
  for (int c = 0; c < n; ++c) {
    const float S = orc_f16_to_f32(st[2 * c]), Cp = orc_f16_to_f32(st[2 * c + 1]);
    const float d = S / 256.0f;
    for (int w = 0; w < 4; ++w)
      for (int b = 0; b < 4; ++b) {
        const float u = (float)((dw[c * 4 + w] >> (8 * b)) & 255u);
        out[(4 * w + kPerm4[b]) * n + c] = (u * d + S) + Cp;
      }
  }
}

/* ---- kv4a16 ----------------------------------------------------------------------------------------------------------- */

void orc_kv4_hadamard256(float* x) {
  for (int h = 1; h < 256; h <<= 1)
    for (int i = 0; i < 256; ++i)
      if (!(i & h)) {
        const float a = x[i], b = x[i ^ h];
        x[i] = a + b;
        x[i ^ h] = a - b;
      }
}

void orc_kv4_quant_k(const float* k, const float* mean, int32_t n_heads, uint32_t* dw, uint16_t* sc) {
  for (int hd = 0; hd < n_heads; ++hd) {
    float x[256];
    for (int i = 0; i < 256; ++i) x[i] = trunc_f16(k[hd * 256 + i]) - mean[hd * 256 + i];
    orc_kv4_hadamard256(x);
    for (int i = 0; i < 256; ++i) x[i] = x[i] * 0.0625f; /* 1 / sqrt(256) */
    for (int g = 0; g < 8; ++g) {
      const float* xr = x + 32 * g;
      float lo = xr[0], hi = xr[0];
      for (int i = 1; i < 32; ++i) lo = fminf(lo, xr[i]), hi = fmaxf(hi, xr[i]);
      const float s0 = (hi - lo) / 15.0f;
      const float s = s0 > 0.0f ? s0 : 1.0f;
      const float inv = 1.0f / s;
      for (int c = 0; c < 4; ++c) {
        uint32_t w = 0;
        for (int i = 0; i < 8; ++i) {
          const float r = fminf(fmaxf(rintf((xr[8 * c + i] - lo) * inv), 0.0f), 15.0f);
          w |= (code_of(r) & 15u) << (4 * (i / 2) + (i % 2 ? 16 : 0));
        }
        dw[hd * 32 + g * 4 + c] = w;
      }
      const float S0 = s * 16.0f;
      sc[2 * (hd * 8 + g)] = orc_f32_to_f16(S0);
      sc[2 * (hd * 8 + g) + 1] = orc_f32_to_f16(lo - S0);
    }
  }
}

void orc_kv4_deq_k(const uint32_t* dw, const uint16_t* sc, int32_t n_heads, float* out) {
  for (int g = 0; g < n_heads * 8; ++g) {
    const float S = orc_f16_to_f32(sc[2 * g]), C = orc_f16_to_f32(sc[2 * g + 1]);
    const float d = S / 16.0f, lo = C + S;
    for (int c = 0; c < 4; ++c)
      for (int i = 0; i < 8; ++i) {
        const float u = (float)((dw[g * 4 + c] >> (4 * (i / 2) + (i % 2 ? 16 : 0))) & 15u);
        out[g * 32 + 8 * c + i] = u * d + lo;
      }
  }
}

static int key_of_nibble4(int w, int p) { return 8 * w + (p < 4 ? 2 * p : 2 * (p - 4) + 1); }

void orc_kv4_quant_vtile(const uint16_t* v, int32_t n, uint32_t* dw, uint16_t* st) {
  for (int c = 0; c < n; ++c) {
    float x[16], mx, mn;
    for (int j = 0; j < 16; ++j) x[j] = orc_f16_to_f32(v[j * n + c]);
    mx = mn = x[0];
    for (int j = 1; j < 16; ++j) mx = fmaxf(mx, x[j]), mn = fminf(mn, x[j]);
    const float cen = (mx + mn) * 0.5f;
    const float s0 = (mx - mn) / 14.0f;
    const float s = s0 > 0.0f ? s0 : 1.0f;
    const float sf = trunc_f16(s), cf = trunc_f16(cen);
    const float inv = 1.0f / sf;
    for (int w = 0; w < 2; ++w) {
      uint32_t word = 0;
      for (int p = 0; p < 8; ++p) {
        const float q = (x[key_of_nibble4(w, p)] - cf) * inv;
        const float r = fminf(fmaxf(rintf(q) + 7.0f, 0.0f), 14.0f);
        word |= (code_of(r) & 15u) << (4 * p);
      }
      dw[c * 2 + w] = word;
    }
    st[2 * c] = orc_f32_to_f16(sf * 16.0f);
    st[2 * c + 1] = orc_f32_to_f16(cf + sf * -23.0f); /* sf * 23 is exact in f32 (sf has 11 bits) */
  }
}

void orc_kv4_deq_vtile(const uint32_t* dw, const uint16_t* st, int32_t n, float* out) {
  for (int c = 0; c < n; ++c) {
    const float S = orc_f16_to_f32(st[2 * c]), Cp = orc_f16_to_f32(st[2 * c + 1]);
    const float d = S / 16.0f;
    for (int w = 0; w < 2; ++w)
      for (int p = 0; p < 8; ++p) {
        const float u = (float)((dw[c * 2 + w] >> (4 * p)) & 15u);
        out[key_of_nibble4(w, p) * n + c] = (u * d + S) + Cp;
      }
  }
}

void orc_kv4_rotate_q(const float* q, float* out) {
  float x[256];
  memcpy(x, q, sizeof(x));
  orc_kv4_hadamard256(x);
  for (int i = 0; i < 256; ++i) out[i] = x[i] * 0.0625f;
}

void orc_kv8_kmean(const float* k, int32_t n_rows, int32_t W, float* mean) {
  for (int c = 0; c < W; ++c) {
    float grp[8];
    for (int g = 0; g < 8; ++g) { /* row group g sums rows g, g + 8, ... in order */
      float a = 0.0f;
      for (int r = g; r < n_rows; r += 8) a = a + trunc_f16(k[(size_t)r * W + c]);
      grp[g] = a;
    }
    float sum = 0.0f;
    for (int g = 0; g < 8; ++g) sum = sum + grp[g];
    mean[c] = sum / (float)n_rows;
  }
}

static int kq_row_dwords(const orc_kv8_geometry* g) { return g->n_kv_heads * (g->k_bits == 4 ? 32 : 64); }
static int ks_row_dwords(const orc_kv8_geometry* g) { return g->n_kv_heads * (g->k_bits == 4 ? 8 : 2); }
static int vq_dwords(const orc_kv8_geometry* g) { return g->v_bits == 4 ? 2 : 4; } /* per (tile, dim) */

static int page_of(const orc_kv8_geometry* g, const int32_t* row, int32_t pos) {
  int pg = row[pos / 256];
  if (pg < 0) pg = 0;
  if (pg > g->n_pages - 1) pg = g->n_pages - 1;
  return pg;
}

/* quantizes the 16 x W tile `tile` (f16 bits, [16][W]) into physical tile `pt` of every head */
static void store_vtile(const orc_kv8_geometry* g, const orc_kv8_pools* p, const uint16_t* tile, int pt) {
  const int H = g->n_kv_heads, W = H * 256;
  const size_t tiles = (size_t)g->n_pages * 16;
  const size_t nw = (size_t)vq_dwords(g);
  uint32_t* dw = (uint32_t*)malloc(sizeof(uint32_t) * (size_t)W * 4);
  uint16_t* st = (uint16_t*)malloc(sizeof(uint16_t) * (size_t)W * 2);
  if (g->v_bits == 4) orc_kv4_quant_vtile(tile, W, dw, st);
  else orc_kv8_quant_vtile(tile, W, dw, st);
  for (int h = 0; h < H; ++h) {
    memcpy(p->vq + (((size_t)h * tiles + (size_t)pt) * 256) * nw, dw + (size_t)h * 256 * nw, sizeof(uint32_t) * 256 * nw);
    memcpy(p->vs + ((size_t)h * tiles + (size_t)pt) * 256, st + (size_t)h * 256 * 2, sizeof(uint32_t) * 256);
  }
  free(dw);
  free(st);
}

void orc_kv8_append(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* table, int32_t stride,
                    const int32_t* start_pos, const int32_t* n_valid, int32_t n_seqs, int32_t n_new,
                    const float* k_src, const float* v_src) {
  const int H = g->n_kv_heads, W = H * 256;
  const int64_t cap = (int64_t)stride * 256;
  uint16_t* tile = (uint16_t*)malloc(sizeof(uint16_t) * 16 * (size_t)W);
  for (int s = 0; s < n_seqs; ++s) {
    const int32_t* row = table + (size_t)s * stride;
    const int64_t p0 = start_pos[s];
    int64_t nv = n_valid != NULL ? n_valid[s] : n_new;
    if (nv > n_new) nv = n_new;
    if (p0 < 0) continue;
    if (p0 + nv > cap) nv = cap - p0; /* positions past the table are not written */
    if (nv <= 0) continue;
    const float* ks = k_src + (size_t)s * n_new * W;
    const float* vs = v_src + (size_t)s * n_new * W;
    const float* mean = p->km + (size_t)page_of(g, row, 0) * W;
    for (int64_t i = 0; i < nv; ++i) {
      const int64_t pos = p0 + i, r = (int64_t)page_of(g, row, (int32_t)pos) * 256 + pos % 256;
      uint32_t* dw = p->kq + (size_t)r * kq_row_dwords(g);
      uint16_t* sc = (uint16_t*)(p->ks + (size_t)r * ks_row_dwords(g));
      if (g->k_bits == 4) orc_kv4_quant_k(ks + (size_t)i * W, mean, H, dw, sc);
      else orc_kv8_quant_k(ks + (size_t)i * W, mean, W / 128, dw, sc);
    }
    if (n_new == 1) { /* the decoder's vappend */
      const int pg = page_of(g, row, (int32_t)p0), key = (int)(p0 % 16);
      uint16_t* vo = p->vo + (size_t)pg * W * 16;
      for (int c = 0; c < W; ++c) vo[(size_t)c * 16 + key] = orc_f32_to_f16(vs[c]);
      if (key == 15) {
        for (int j = 0; j < 16; ++j)
          for (int c = 0; c < W; ++c) tile[(size_t)j * W + c] = vo[(size_t)c * 16 + j];
        store_vtile(g, p, tile, pg * 16 + (int)((p0 / 16) % 16));
      }
      continue;
    }
    const int64_t last = p0 + nv - 1;
    for (int64_t t = p0 / 16; t <= last / 16; ++t) { /* the prefill's vq8 over every tile the chunk touches */
      const int pg = page_of(g, row, (int32_t)(16 * t));
      uint16_t* vo = p->vo + (size_t)pg * W * 16;
      for (int j = 0; j < 16; ++j) {
        const int64_t pos = 16 * t + j;
        for (int c = 0; c < W; ++c) {
          uint16_t x;
          if (pos < p0) x = vo[(size_t)c * 16 + j];                        /* appended earlier: in the open tile */
          else x = orc_f32_to_f16(vs[(size_t)((pos <= last ? pos : last) - p0) * W + c]); /* past the end: the last */
          tile[(size_t)j * W + c] = x;
        }
      }
      store_vtile(g, p, tile, pg * 16 + (int)(t % 16));
      if (t == last / 16) { /* vseed: the newest tile stays open, keys past the last real token zero */
        for (int j = 0; j < 16; ++j) {
          const int64_t pos = 16 * t + j;
          if (pos < p0) continue;
          for (int c = 0; c < W; ++c) vo[(size_t)c * 16 + j] = pos <= last ? tile[(size_t)j * W + c] : 0;
        }
      }
    }
  }
  free(tile);
}

static void dense(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* row, int32_t n, float* Kd, float* Vd,
                  int as_f16) {
  const int H = g->n_kv_heads, W = H * 256;
  const size_t tiles = (size_t)g->n_pages * 16;
  const int curt = n > 0 ? (n - 1) / 16 : 0;
  float out[16 * 256];
  for (int pos = 0; pos < n; ++pos) {
    const size_t r = (size_t)page_of(g, row, pos) * 256 + (size_t)(pos % 256);
    const uint32_t* dw = p->kq + r * kq_row_dwords(g);
    const uint16_t* sc = (const uint16_t*)(p->ks + r * ks_row_dwords(g));
    if (!as_f16 && g->k_bits == 4) {
      orc_kv4_deq_k(dw, sc, H, Kd + (size_t)pos * W);
    } else if (!as_f16) {
      orc_kv8_deq_k(dw, sc, W / 128, Kd + (size_t)pos * W);
    } else if (g->k_bits == 4) { /* yah_kdeq4: f16(1 + u / 16) * S + C, one f16 fma (gen_attn_fa.py:4652-4700) */
      for (int i = 0; i < W / 8; ++i)
        for (int e = 0; e < 8; ++e) {
          const double f = 1.0 + (double)((dw[i] >> (4 * (e / 2) + (e % 2 ? 16 : 0))) & 15u) / 16.0;
          const int gi = (8 * i) / 32;
          const double v = fma(f, (double)orc_f16_to_f32(sc[2 * gi]), (double)orc_f16_to_f32(sc[2 * gi + 1]));
          Kd[(size_t)pos * W + 8 * i + e] = orc_f16_to_f32(f64_to_f16(v));
        }
    } else {
      for (int i = 0; i < W / 4; ++i)
        for (int b = 0; b < 4; ++b) {
          const double f = 1.0 + (double)((dw[i] >> (8 * b)) & 255u) / 256.0;
          const int hh = (4 * i) / 128;
          const double v = fma(f, (double)orc_f16_to_f32(sc[2 * hh]), (double)orc_f16_to_f32(sc[2 * hh + 1]));
          Kd[(size_t)pos * W + 4 * i + kPerm4[b]] = orc_f16_to_f32(f64_to_f16(v));
        }
    }
  }
  for (int t = 0; 16 * t < n; ++t) {
    const int pg = page_of(g, row, 16 * t), pt = pg * 16 + t % 16;
    const int keys = n - 16 * t < 16 ? n - 16 * t : 16;
    for (int h = 0; h < H; ++h) {
      if (!as_f16 && t == curt) { /* the newest tile is read from the open f16 tile */
        const uint16_t* vo = p->vo + ((size_t)pg * W + (size_t)h * 256) * 16;
        for (int j = 0; j < keys; ++j)
          for (int c = 0; c < 256; ++c) Vd[(size_t)(16 * t + j) * W + h * 256 + c] = orc_f16_to_f32(vo[(size_t)c * 16 + j]);
        continue;
      }
      const uint32_t* dw = p->vq + (((size_t)h * tiles + (size_t)pt) * 256) * (size_t)vq_dwords(g);
      const uint16_t* st = (const uint16_t*)(p->vs + ((size_t)h * tiles + (size_t)pt) * 256);
      if (!as_f16 && g->v_bits == 4) {
        orc_kv4_deq_vtile(dw, st, 256, out);
      } else if (!as_f16) {
        orc_kv8_deq_vtile(dw, st, 256, out);
      } else if (g->v_bits == 4) { /* yah_vdeq4: f16(1 + u / 16) * S + C' */
        for (int c = 0; c < 256; ++c)
          for (int w = 0; w < 2; ++w)
            for (int pn = 0; pn < 8; ++pn) {
              const double f = 1.0 + (double)((dw[c * 2 + w] >> (4 * pn)) & 15u) / 16.0;
              const double v = fma(f, (double)orc_f16_to_f32(st[2 * c]), (double)orc_f16_to_f32(st[2 * c + 1]));
              out[key_of_nibble4(w, pn) * 256 + c] = orc_f16_to_f32(f64_to_f16(v));
            }
      } else {
        for (int c = 0; c < 256; ++c)
          for (int w = 0; w < 4; ++w)
            for (int b = 0; b < 4; ++b) {
              const double f = 1.0 + (double)((dw[c * 4 + w] >> (8 * b)) & 255u) / 256.0;
              const double v = fma(f, (double)orc_f16_to_f32(st[2 * c]), (double)orc_f16_to_f32(st[2 * c + 1]));
              out[(4 * w + kPerm4[b]) * 256 + c] = orc_f16_to_f32(f64_to_f16(v));
            }
      }
      for (int j = 0; j < keys; ++j)
        memcpy(Vd + (size_t)(16 * t + j) * W + h * 256, out + j * 256, sizeof(float) * 256);
    }
  }
}

void orc_kv8_dense(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* table_row, int32_t n_tokens,
                   float* Kd, float* Vd) {
  dense(g, p, table_row, n_tokens, Kd, Vd, 0);
}

void orc_kv8_dense_f16(const orc_kv8_geometry* g, const orc_kv8_pools* p, const int32_t* table_row, int32_t n_tokens,
                       float* Kd, float* Vd) {
  dense(g, p, table_row, n_tokens, Kd, Vd, 1);
}
