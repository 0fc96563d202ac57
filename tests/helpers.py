"""Shared test helpers: seeded inputs of the benchmark configurations, an independent numpy reading of the pool
layout documented in include/yahkv.h, and the float64 closed-form attention the reference's own checker uses
(engine/gpu/loom/tools/dattn_q_check.py:193-203)."""
import numpy as np

import oracle


def blocks_per_head(g):
    return g.head_dim // 32


def make_tables(rng, seq_pages, n_pages, stride=None):
    """One shared pool, pages handed out from one global shuffle (dattn_q_check.py:151 scrambles its table too)."""
    perm = rng.permutation(n_pages).astype(np.int32)
    stride = stride or max(seq_pages)
    table = np.zeros((len(seq_pages), stride), np.int32)
    o = 0
    for s, n in enumerate(seq_pages):
        table[s, :n] = perm[o:o + n]
        o += n
    assert o <= n_pages
    return table


def logical_blocks(arrs, g, table_row, n_tokens):
    """(scale bits u16 [n][H][NB], codes [n][H][NB][32] int32) of K and V read straight from the documented layout."""
    H, D, PT, NB = g.n_kv_heads, g.head_dim, g.page_tokens, g.head_dim // 32
    P = g.n_pages
    pos = np.arange(n_tokens)
    page, t = np.asarray(table_row)[pos // PT], pos % PT
    ks = arrs["ks"].reshape(P, H, PT, NB)[page, :, t, :]                       # [n][H][NB]
    vs = arrs["vs"].reshape(P, H, NB, PT)[page, :, :, t]
    if g.format == 8:
        kc = arrs["kq"].reshape(P, H, NB, PT, 32)[page, :, :, t, :].view(np.int8).astype(np.int32)
        vc = arrs["vq"].reshape(P, H, D, PT)[page, :, :, t].reshape(n_tokens, H, NB, 32).view(np.int8).astype(np.int32)
    else:
        kb = arrs["kq"].reshape(P, H, NB, PT, 16)[page, :, :, t, :]
        vb = arrs["vq"].reshape(P, H, NB, 16, PT)[page, :, :, :, t]
        kc = np.concatenate([kb & 0xF, kb >> 4], -1).astype(np.int32) - 8
        vc = np.concatenate([vb & 0xF, vb >> 4], -1).astype(np.int32) - 8
    return (ks, kc), (vs, vc)


def dequant(scale_bits, codes):
    d = np.ascontiguousarray(scale_bits).view(np.float16).astype(np.float32)
    y = d[..., None] * codes.astype(np.float32)                               # f32 product, as gguf_quant.cpp:72-75
    return y.reshape(*y.shape[:-2], -1)                                       # [n][H][D]


def closed_form(Kd, Vd, q, scale, gate=None):
    """softmax(q K^T * scale) V in float64 for one sequence. Kd/Vd [n][H][D] f32, q [NQ][D]."""
    n, H, D = Kd.shape
    NQ = q.shape[0]
    G = NQ // H
    out = np.zeros((NQ, D))
    for h in range(NQ):
        kv = h // G
        s = Kd[:, kv].astype(np.float64) @ q[h].astype(np.float64) * scale
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h] = p @ Vd[:, kv].astype(np.float64)
        if gate is not None:
            out[h] /= 1.0 + np.exp(-gate[h].astype(np.float64))
    return out


def rel_err(got, want):
    """The reference checker's metric: max |got - want| / max |want| (dattn_q_check.py:205)."""
    return float(np.abs(got - want).max() / np.abs(want).max())


def to_f16_f32(x):
    return np.asarray(x).astype(np.float16).astype(np.float32)


def to_bf16_f32(x):
    x = np.ascontiguousarray(x, np.float32)
    return oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(x)).reshape(x.shape)


def bf16_bits(x):
    x = np.ascontiguousarray(x, np.float32)
    return oracle.f32_to_bf16_bits(x).reshape(x.shape)
