#!/usr/bin/env python3
"""Writes tests/golden/kv8a16_vectors.npz: inputs and the outputs of the REFERENCE's own numpy model of its kv8a16
KV format: quant_k, deq_k, quant_vtile, deq_vtile of engine/gpu/loom/tools/dattn_q_check.py:61-137, imported from
/root/reference where it lies. Nothing of the reference is copied: the .npz holds plain arrays (data only, loaded with
allow_pickle=False), and this script never travels to the GPU box's runs.

Run in the authoring container, where the reference tree exists:  python tests/golden/make_kv8a16_vectors.py

Contents
  k_in f32 [n][1024], k_mean f32 [n][1024]  ->  k_dw u32 [n][256], k_sc u16 [n][16] (f16 bits), k_deq f32 [n][1024]
      single K rows (4 kv heads x 256 dims) through quant_k(.., 8) and deq_k: random rows and means, all-zero halves
      (s <= 0 -> 1), products on round-half-even ties, outliers, scales beyond the f16 range at both ends, sources that
      f16 truncation changes
  v_in f16 [n][16][64]  ->  v_dw u32 [n][64][4], v_st u16 [n][64][2], v_deq f32 [n][16][64]
      16-key V tiles of 64 channels through quant_vtile(.., 8) and deq_vtile: random tiles, tiles of equal values,
      two-valued tiles, ties, large magnitudes
  The checker's own recipe (dattn_q_check.py:140-256; rng 5, T 1024, pos 700, scrambled page table), prefix rc_:
      rc_ptab, rc_m, rc_q, rc_gate and sha256 digests of K and V (the tests draw them again from the seed and
      compare the digests), rc_ks / rc_vs / rc_vopen in full, rc_kq_sha / rc_vq_sha digests of the code pools plus
      sampled rows (rc_kq_rows_idx, rc_kq_rows; rc_vq_tiles_idx, rc_vq_tiles), rc_ref (attention over the dequantized
      model, float64, :193-203) and rc_exact (over the f16 K / V); then the append cases of :210-250:
      rc_kx + rc_k2_dw / rc_k2_sc at position 517, and rc_vx / rc_vo / rc_vo_out / rc_v3_dw / rc_v3_st for the two V
      appends (mid-tile at 16 * 37 + 9, tile-closing at 16 * 37 + 15).
"""
import hashlib
import os
import sys

import numpy as np

REF_TOOLS = "/root/reference/engine/gpu/loom/tools"
sys.dont_write_bytecode = True
sys.path.insert(0, REF_TOOLS)
import dattn_q_check as R  # noqa: E402  (the reference's checker module: numpy model only, main() is not run)

f32, f16 = np.float32, np.float16
OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kv8a16_vectors.npz")


def sha(a):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), np.uint8).copy()


def k_rows():
    rng = np.random.default_rng(811)
    rows, means = [], []

    def add(k, m=None):
        rows.append(np.asarray(k, f32).reshape(1024))
        means.append(np.zeros(1024, f32) if m is None else np.asarray(m, f32).reshape(1024))

    for _ in range(12):                                        # the recipe's distribution: K ~ N(m, 1), m ~ 0.5 N(0, 1)
        m = (0.5 * rng.standard_normal(1024)).astype(f32)
        add(rng.standard_normal(1024) + m, m)
    for e in (-6, -3, 2, 4):                                   # other magnitudes
        add(rng.standard_normal(1024) * 10.0 ** e, (rng.standard_normal(1024) * 10.0 ** e).astype(f32))
    add(np.zeros(1024))                                        # every half dead: s -> 1, codes 128, scales (256, -384)
    z = rng.standard_normal(1024)
    z[128:256] = 0.0                                           # one dead half among live ones
    z[512:640] = 0.0
    add(z)
    m = rng.standard_normal(1024).astype(f16).astype(f32)
    add(m, m)                                                  # K == mean exactly: x = 0 everywhere
    # amax = 127 -> s = 1, inv = 1: x lands exactly on halves; rne goes to the even code, lround would not
    t = np.zeros(1024)
    t[0] = 127.0
    t[1:17] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 126.5, -126.5, 100.5, -100.5, 3.5, -3.5, 64.5, -64.5]
    t[128] = -127.0                                            # second half: the extreme is negative
    t[129:137] = [0.5, -0.5, 1.5, -1.5, 126.5, -126.5, 2.5, -2.5]
    add(t)
    # amax = 254 -> s = 2, inv = 0.5: odd values land on halves as well
    t = np.zeros(1024)
    t[256] = 254.0
    t[257:265] = [1.0, 3.0, 5.0, -1.0, -3.0, -5.0, 253.0, -253.0]
    add(t)
    # a single outlier per half, the rest small (SageAttention's case)
    t = rng.standard_normal(1024) * 0.01
    t[::128] = [30.0, -30.0, 55.5, -0.75, 1000.0, -1000.0, 7.0, -7.0]
    add(t)
    # scales at the ends of the f16 range: 256 s overflows to inf / underflows to a subnormal or zero
    t = np.zeros(1024)
    t[0], t[1] = 60000.0, -30000.0                             # s = 472.4: 256 s = 1.2e5 -> f16 inf
    t[128], t[129] = 1e-6, -5e-7                               # s = 7.9e-9: 256 s = 2e-6 (f16 subnormal)
    t[256], t[257] = 6e-8, 0.0                                 # one f16 subnormal step
    t[384], t[385] = 200.0, -100.0
    add(t)
    # sources that are not f16 values: the quantizer truncates to f16 first (round to nearest even)
    t = rng.standard_normal(1024) * (1 + 2.0 ** -12)
    t[5], t[6], t[7] = 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 65519.0    # ties of the f16 rounding; largest that stays finite
    add(t, (0.25 * rng.standard_normal(1024)).astype(f32))
    # mean much larger than the spread (what the mean is for)
    m = (20.0 * rng.standard_normal(1024)).astype(f32)
    add(m + 0.05 * rng.standard_normal(1024), m)
    return np.stack(rows), np.stack(means)


def v_tiles():
    rng = np.random.default_rng(812)
    tiles = []

    def add(v):
        tiles.append(np.asarray(v, f32).astype(f16).reshape(16, 64))

    for _ in range(10):
        add(rng.standard_normal((16, 64)))
    for e in (-4, -2, 2, 4):
        add(rng.standard_normal((16, 64)) * 10.0 ** e)
    add(np.zeros((16, 64)))                                    # s0 = 0 -> s = 1, every code 128
    add(np.full((16, 64), 3.25))                               # equal values off zero
    add(np.tile(rng.standard_normal((1, 64)), (16, 1)))        # every channel constant over its keys
    t = np.zeros((16, 64))
    t[::2] = 1.0                                               # two-valued: codes 1 and 255
    t[1::2] = -1.0
    add(t)
    # range 254 -> s = 1, centre 0: halves land on ties
    t = np.zeros((16, 64))
    t[0], t[1] = 127.0, -127.0
    t[2:16] = np.array([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 126.5, -126.5, 100.5, -100.5, 3.5, -3.5])[:, None]
    add(t)
    # centre not an f16 value: c rounds, and the codes of the extremes clip at 1 / 255 or not
    t = rng.standard_normal((16, 64))
    t[0] = 1000.0 + rng.uniform(0, 1, 64)
    t[1] = 999.0 - rng.uniform(0, 1, 64)
    add(t)
    t = rng.standard_normal((16, 64)) * 1e-3 + 300.0           # spread far below the centre's f16 step
    add(t)
    t = np.zeros((16, 64))
    t[0], t[1] = 60000.0, -60000.0                             # range beyond f16: 256 s overflows
    t[2:] = rng.uniform(-60000, 60000, (14, 64))
    add(t)
    t = rng.standard_normal((16, 64))
    t[:, ::2] *= 50.0                                          # neighbouring channels on very different scales
    add(t)
    return np.stack(tiles)


def recipe():
    """dattn_q_check.py:140-256 for bits 8, T 1024, pos 700, in its order of random draws."""
    T, pos, bits = 1024, 700, 8
    rng = np.random.default_rng(5)
    npg, tiles, n = T // 256, T // 16, pos + 1
    ptab = rng.permutation(npg).astype(np.int32)
    prow = lambda p: ptab[p // 256] * 256 + p % 256
    m = (0.5 * rng.standard_normal(1024)).astype(f32)
    K = (rng.standard_normal((T, 1024)) + m).astype(f16)
    V = rng.standard_normal((T, 1024)).astype(f16)
    q = (0.3 * rng.standard_normal((24, 256))).astype(f32)
    gate = rng.standard_normal((24, 256)).astype(f32)
    kq = np.zeros((T, 256), np.uint32)
    ks = np.zeros((T, 16), f16)
    Kd = np.zeros((T, 1024), f32)
    for p in range(T):
        dw, sc = R.quant_k(K[p].astype(f32), m, bits)
        kq[prow(p)], ks[prow(p)] = dw, sc
        Kd[p] = R.deq_k(dw, sc, bits)
    vq = np.zeros((4, tiles, 256, 4), np.uint32)
    vs = np.zeros((4, tiles, 256, 2), f16)
    Vd = V.astype(f32).copy()
    curt = pos // 16
    for t in range(curt):
        dw, st = R.quant_vtile(V[16 * t:16 * t + 16], bits)
        pt = ptab[t // 16] * 16 + t % 16
        vq[:, pt], vs[:, pt] = dw.reshape(4, 256, 4), st.reshape(4, 256, 2)
        Vd[16 * t:16 * t + 16] = R.deq_vtile(dw, st, bits)
    vopen = np.zeros((1024, 16), f16)
    nk = pos - 16 * curt + 1
    vopen[:, :nk] = V[16 * curt:pos + 1].T
    vopen[:, nk:] = 7.0                                        # stale keys past pos: masked

    def attn(Kx, Vx, qx):
        ref = np.zeros((24, 256))
        for hh in range(24):
            kv = hh // 6
            s = Kx[:n, kv * 256:kv * 256 + 256].astype(np.float64) @ qx[hh].astype(np.float64) / 16.0
            pr = np.exp(s - s.max())
            pr /= pr.sum()
            ref[hh] = (pr @ Vx[:n, kv * 256:kv * 256 + 256].astype(np.float64)) / (1.0 + np.exp(-gate[hh].astype(np.float64)))
        return ref
    ref = attn(Kd, Vd, q)
    exact = attn(K.astype(f32) - m, V, q)
    out = dict(rc_T=np.int32(T), rc_pos=np.int32(pos), rc_ptab=ptab, rc_m=m, rc_q=q, rc_gate=gate, rc_K_sha=sha(K),
               rc_V_sha=sha(V), rc_ks=ks.view(np.uint16), rc_vs=vs.view(np.uint16), rc_vopen=vopen.view(np.uint16),
               rc_kq_sha=sha(kq), rc_vq_sha=sha(vq), rc_Kd_sha=sha(Kd), rc_Vd_sha=sha(Vd), rc_ref=ref, rc_exact=exact)
    rows = np.sort(np.random.default_rng(6).choice(T, 40, replace=False)).astype(np.int32)     # physical rows
    out["rc_kq_rows_idx"], out["rc_kq_rows"] = rows, kq[rows]
    tls = np.sort(np.random.default_rng(7).choice(tiles, 6, replace=False)).astype(np.int32)   # physical tiles
    out["rc_vq_tiles_idx"], out["rc_vq_tiles"] = tls, vq[:, tls]
    # kappend at p2 (:210-225)
    p2 = min(517, T - 1)
    kx = (rng.standard_normal(1024) + m).astype(f32)
    dw, sc = R.quant_k(kx, m, bits)
    out["rc_p2"], out["rc_kx"], out["rc_k2_dw"], out["rc_k2_sc"] = np.int32(p2), kx, dw, sc.view(np.uint16)
    # vappend: a mid-tile key (open tile only), then a tile's 16th key (quantize) (:227-250)
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
            out["rc_v3_dw"], out["rc_v3_st"] = dw.reshape(4, 256, 4), st.reshape(4, 256, 2).view(np.uint16)
    return out


def main():
    k_in, k_mean = k_rows()
    k_dw, k_sc, k_deq = [], [], []
    for k, m in zip(k_in, k_mean):
        with np.errstate(all="ignore"):
            dw, sc = R.quant_k(k, m, 8)
            k_dw.append(dw), k_sc.append(sc.view(np.uint16)), k_deq.append(R.deq_k(dw, sc, 8))
    v_in = v_tiles()
    v_dw, v_st, v_deq = [], [], []
    for v in v_in:
        with np.errstate(all="ignore"):
            dw, st = R.quant_vtile(v, 8)
            v_dw.append(dw), v_st.append(st.view(np.uint16)), v_deq.append(R.deq_vtile(dw, st, 8))
    data = dict(k_in=k_in, k_mean=k_mean, k_dw=np.stack(k_dw), k_sc=np.stack(k_sc), k_deq=np.stack(k_deq).astype(f32),
                v_in=v_in.view(np.uint16), v_dw=np.stack(v_dw), v_st=np.stack(v_st), v_deq=np.stack(v_deq).astype(f32))
    data.update(recipe())
    np.savez_compressed(OUT, **data)
    print(OUT, os.path.getsize(OUT), "bytes;", len(k_in), "K rows,", len(v_in), "V tiles")


if __name__ == "__main__":
    main()
