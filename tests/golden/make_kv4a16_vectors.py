#!/usr/bin/env python3
"""Writes tests/golden/kv4a16_vectors.npz: inputs and the outputs of the REFERENCE's own numpy model of its kv4a16 KV
format: quant_k, deq_k, quant_vtile, deq_vtile with bits = 4 and the Hadamard matrix H of
engine/gpu/loom/tools/dattn_q_check.py:52-137, imported from /root/reference where it lies. Nothing of the reference
is copied: the .npz holds plain arrays (data only, loaded with allow_pickle=False), and this script never travels to
the GPU box's runs.

Run in the authoring container, where the reference tree exists:  python tests/golden/make_kv4a16_vectors.py

The numpy model rotates K in float64 (x @ H.T / 16, then to f32); the reference's kernel, and the oracle here, run the
butterflies in f32 in a fixed order. The two agree bit for bit wherever every partial sum is exact, so the K rows
come in two kinds:
  kx_in f32 [n][1024] (mean zero)  ->  kx_dw u32 [n][128], kx_sc u16 [n][64], kx_deq f32 [n][1024]
      "exact" rows: small multiples of 1/16 made as H (wanted rotated values) / 16, so that the rotation is exact in
      any order and the codes, scales and decoded values are pinned bit for bit: ties of the rounding (range 15 -> s = 1),
      dead groups (s0 = 0 -> 1), a range that is no power of two, groups off zero, negative lows, clipping ends
  kr_in, kr_mean f32 [n][1024]     ->  kr_dw, kr_sc, kr_deq
      random rows and means (the recipe's distribution and other magnitudes): pinned within the rounding of the
      rotation (a code may move by one step where a value sits on a rounding boundary)
  v_in f16 [n][16][64]  ->  v_dw u32 [n][64][2], v_st u16 [n][64][2], v_deq f32 [n][16][64]   (bit for bit)
  had_in f32 [8][256] -> had_out f64 [8][256] = in @ H.T (the matrix itself, for the butterfly's sign and index order)
  The checker's own recipe (dattn_q_check.py:140-256 with bits 4; rng 5, T 1024, pos 700, scrambled page table),
  prefix rc_: as in kv8a16_vectors.npz, with rc_qr (the rotated query, float64) besides rc_q.
"""
import os
import sys

import numpy as np

sys.dont_write_bytecode = True
sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
import make_kv8a16_vectors as M8  # noqa: E402  (the 8-bit script: imports the reference's module as R)

R, sha = M8.R, M8.sha
f32, f16 = np.float32, np.float16
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kv4a16_vectors.npz")


def exact_rows():
    rng = np.random.default_rng(411)
    rows = []

    def add(xr):
        """xr: wanted rotated values [4][256] (integers or multiples of 1/2); the row is H xr / 16"""
        xr = np.asarray(xr, np.float64).reshape(4, 256)
        x = xr @ R.H.T / 16.0
        assert np.abs(x).max() < 128 and np.array_equal(x * 16, np.round(x * 16)), "not exact in f16"
        assert np.array_equal(x.astype(f16).astype(np.float64), x)
        rows.append(x.astype(f32).reshape(1024))

    # range 15 -> s = 1: halves land on ties, rne goes to the even code
    t = np.zeros((4, 256))
    t[0, :32] = [0, 15, 0.5, 1.5, 2.5, 3.5, 13.5, 14.5, 7.5, 8.5, 1, 2, 3, 4, 5, 6] + [0] * 16
    t[1, 32:64] = [-5, 10, -4.5, -3.5, -2.5, 9.5, 8.5, 0.5, -0.5, 1.5] + [0] * 22      # lo = -5
    t[2, 64:96] = 3.0                                                                   # a constant group off zero: s0 = 0 -> 1
    t[3, 96:128] = np.arange(32) % 16                                                   # every code once or twice
    add(t)
    # range 30 -> s = 2, inv = 0.5: odd values land on halves
    t = np.zeros((4, 256))
    t[0, :32] = [0, 30] + list(range(1, 31))
    t[1, 128:160] = [-30, 0] + [-x for x in range(1, 31)]
    add(t)
    # a range that is no power of two (7 -> s = 7 / 15): the products round
    t = np.zeros((4, 256))
    t[0, :32] = [0, 7] + [(x % 8) for x in range(30)]
    t[2, 224:256] = [-3, 4] + [((x * 5) % 8) - 3 for x in range(30)]
    add(t)
    for _ in range(5):                                         # random small integers in every group
        add(rng.integers(-6, 7, (4, 256)))
    add(np.zeros((4, 256)))                                    # the zero row: every group dead
    t = np.zeros((4, 256))
    t[:, ::32] = [[40, -40, 17, -3, 8, 1, -1, 25]] * 4         # one outlier per group
    add(t)
    return np.stack(rows)


def random_rows():
    rng = np.random.default_rng(412)
    rows, means = [], []
    for _ in range(10):
        m = (0.5 * rng.standard_normal(1024)).astype(f32)
        rows.append((rng.standard_normal(1024) + m).astype(f32)), means.append(m)
    for e in (-4, -2, 2):
        rows.append((rng.standard_normal(1024) * 10.0 ** e).astype(f32))
        means.append((rng.standard_normal(1024) * 10.0 ** e).astype(f32))
    t = (rng.standard_normal(1024) * 0.05).astype(f32)         # outlier channels, which the rotation spreads
    t[::64] = 20.0
    rows.append(t), means.append(np.zeros(1024, f32))
    return np.stack(rows), np.stack(means)


def v_tiles():
    rng = np.random.default_rng(413)
    tiles = list(M8.v_tiles()[:20])                            # the 8-bit script's random and directed tiles
    t = np.zeros((16, 64))
    t[0], t[1] = 7.0, -7.0                                     # range 14 -> s = 1, centre 0: halves land on ties
    t[2:16] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 6.5, -6.5, 3.5, -3.5, 4.5, -4.5, 5.5, -5.5])[:, None]
    tiles.append(t.astype(f16))
    t = np.zeros((16, 64))
    t[::2], t[1::2] = 1.0, -1.0                                # two-valued: codes 0 and 14
    tiles.append(t.astype(f16))
    tiles.append((rng.standard_normal((16, 64)) * 3 + 100.0).astype(f16))   # centre far from zero
    return np.stack(tiles)


def recipe():
    """dattn_q_check.py:140-256 for bits 4, T 1024, pos 700, in its order of random draws."""
    T, pos, bits = 1024, 700, 4
    rng = np.random.default_rng(5)
    npg, tiles, n = T // 256, T // 16, pos + 1
    ptab = rng.permutation(npg).astype(np.int32)
    prow = lambda p: ptab[p // 256] * 256 + p % 256
    m = (0.5 * rng.standard_normal(1024)).astype(f32)
    K = (rng.standard_normal((T, 1024)) + m).astype(f16)
    V = rng.standard_normal((T, 1024)).astype(f16)
    q = (0.3 * rng.standard_normal((24, 256))).astype(f32)
    gate = rng.standard_normal((24, 256)).astype(f32)
    kq = np.zeros((T, 128), np.uint32)
    ks = np.zeros((T, 64), f16)
    Kd = np.zeros((T, 1024), f32)
    for p in range(T):
        dw, sc = R.quant_k(K[p].astype(f32), m, bits)
        kq[prow(p)], ks[prow(p)] = dw, sc
        Kd[p] = R.deq_k(dw, sc, bits)
    vq = np.zeros((4, tiles, 256, 2), np.uint32)
    vs = np.zeros((4, tiles, 256, 2), f16)
    Vd = V.astype(f32).copy()
    curt = pos // 16
    for t in range(curt):
        dw, st = R.quant_vtile(V[16 * t:16 * t + 16], bits)
        pt = ptab[t // 16] * 16 + t % 16
        vq[:, pt], vs[:, pt] = dw.reshape(4, 256, 2), st.reshape(4, 256, 2)
        Vd[16 * t:16 * t + 16] = R.deq_vtile(dw, st, bits)
    vopen = np.zeros((1024, 16), f16)
    nk = pos - 16 * curt + 1
    vopen[:, :nk] = V[16 * curt:pos + 1].T
    vopen[:, nk:] = 7.0

    def attn(Kx, Vx, qx):
        ref = np.zeros((24, 256))
        for hh in range(24):
            kv = hh // 6
            s = Kx[:n, kv * 256:kv * 256 + 256].astype(np.float64) @ qx[hh].astype(np.float64) / 16.0
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            ref[hh] = (pr @ Vx[:n, kv * 256:kv * 256 + 256].astype(np.float64)) / (1.0 + np.exp(-gate[hh].astype(np.float64)))
        return ref
    qr = q.astype(np.float64) @ R.H.T / 16.0
    ref = attn(Kd, Vd, qr)
    exact = attn(K.astype(f32) - m, V, q)
    out = dict(rc_T=np.int32(T), rc_pos=np.int32(pos), rc_ptab=ptab, rc_m=m, rc_q=q, rc_qr=qr, rc_gate=gate,
               rc_K_sha=sha(K), rc_V_sha=sha(V), rc_kq=kq, rc_ks=ks.view(np.uint16), rc_vs=vs.view(np.uint16),
               rc_vopen=vopen.view(np.uint16), rc_vq_sha=sha(vq), rc_Vd_sha=sha(Vd), rc_ref=ref, rc_exact=exact)
    tls = np.sort(np.random.default_rng(7).choice(tiles, 6, replace=False)).astype(np.int32)
    out["rc_vq_tiles_idx"], out["rc_vq_tiles"] = tls, vq[:, tls]
    p2 = min(517, T - 1)
    kx = (rng.standard_normal(1024) + m).astype(f32)
    dw, sc = R.quant_k(kx, m, bits)
    out["rc_p2"], out["rc_kx"], out["rc_k2_dw"], out["rc_k2_sc"] = np.int32(p2), kx, dw, sc.view(np.uint16)
    for i, p3 in enumerate((16 * 37 + 9, 16 * 37 + 15)):
        vx = rng.standard_normal(1024).astype(f32)
        vo = np.zeros((1024, 16), f16)
        vo[:, :p3 % 16] = rng.standard_normal((1024, p3 % 16)).astype(f16)
        evo = vo.copy()
        evo[:, p3 % 16] = vx.astype(f16)
        out[f"rc_p3_{i}"], out[f"rc_vx_{i}"] = np.int32(p3), vx
        out[f"rc_vo_{i}"], out[f"rc_vo_out_{i}"] = vo.view(np.uint16), evo.view(np.uint16)
        if p3 % 16 == 15:
            dw, st = R.quant_vtile(evo.T, bits)
            out["rc_v3_dw"], out["rc_v3_st"] = dw.reshape(4, 256, 2), st.reshape(4, 256, 2).view(np.uint16)
    return out


def main():
    zero = np.zeros(1024, f32)
    kx_in = exact_rows()
    kx = [R.quant_k(k, zero, 4) for k in kx_in]
    kr_in, kr_mean = random_rows()
    kr = [R.quant_k(k, m, 4) for k, m in zip(kr_in, kr_mean)]
    v_in = v_tiles()
    vv = []
    for v in v_in:
        with np.errstate(all="ignore"):
            vv.append(R.quant_vtile(v, 4))
    had_in = np.random.default_rng(414).standard_normal((8, 256)).astype(f32)
    had_in[0] = 0
    had_in[0, 1] = 1.0                                          # a unit vector: one column of H, signs and order
    had_in[1] = 0
    had_in[1, 130] = 1.0
    data = dict(
        kx_in=kx_in, kx_dw=np.stack([a for a, _ in kx]), kx_sc=np.stack([b.view(np.uint16) for _, b in kx]),
        kx_deq=np.stack([R.deq_k(a, b, 4) for a, b in kx]).astype(f32),
        kr_in=kr_in, kr_mean=kr_mean, kr_dw=np.stack([a for a, _ in kr]), kr_sc=np.stack([b.view(np.uint16) for _, b in kr]),
        kr_deq=np.stack([R.deq_k(a, b, 4) for a, b in kr]).astype(f32),
        v_in=v_in.view(np.uint16), v_dw=np.stack([a for a, _ in vv]), v_st=np.stack([b.view(np.uint16) for _, b in vv]),
        v_deq=np.stack([R.deq_vtile(a, b, 4) for a, b in vv]).astype(f32),
        had_in=had_in, had_out=had_in.astype(np.float64) @ R.H.T)
    data.update(recipe())
    np.savez_compressed(OUT, **data)
    print(OUT, os.path.getsize(OUT), "bytes;", len(kx_in), "exact K rows,", len(kr_in), "random K rows,", len(v_in), "V tiles")


if __name__ == "__main__":
    main()
