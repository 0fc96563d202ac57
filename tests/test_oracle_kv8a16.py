"""The CPU oracle of the reference's own KV format (oracle/kv8_oracle.c) against the reference's numpy model of it:
tests/golden/kv8a16_vectors.npz holds inputs and outputs of quant_k, deq_k, quant_vtile, deq_vtile
(engine/gpu/loom/tools/dattn_q_check.py:61-137) and of the checker's whole recipe (:140-256)."""
import numpy as np
import pytest

import kv8_recipe
from helpers import closed_form, rel_err
from oracle import kv8


@pytest.fixture(scope="module")
def gold():
    return kv8_recipe.golden()


@pytest.fixture(scope="module")
def rc():
    return kv8_recipe.load()


def test_k_rows_bit_exact(gold):
    for i in range(gold["k_in"].shape[0]):
        dw, sc = kv8.quant_k(gold["k_in"][i], gold["k_mean"][i])
        assert np.array_equal(dw, gold["k_dw"][i]), f"K row {i}: codes"
        assert np.array_equal(sc, gold["k_sc"][i]), f"K row {i}: scale pairs"
        assert np.array_equal(kv8.deq_k(gold["k_dw"][i], gold["k_sc"][i]).view(np.uint32),
                              gold["k_deq"][i].view(np.uint32)), f"K row {i}: dequantized values"


def test_v_tiles_bit_exact(gold):
    for i in range(gold["v_in"].shape[0]):
        dw, st = kv8.quant_vtile(gold["v_in"][i])
        assert np.array_equal(dw, gold["v_dw"][i]), f"V tile {i}: codes"
        assert np.array_equal(st, gold["v_st"][i]), f"V tile {i}: stats"
        assert np.array_equal(kv8.deq_vtile(gold["v_dw"][i], gold["v_st"][i]).view(np.uint32),
                              gold["v_deq"][i].view(np.uint32)), f"V tile {i}: dequantized values"


def test_directed_cases_say_what_they_should(gold):
    """The fixture's special rows do exercise the special paths (read off the expected outputs themselves)."""
    sc = gold["k_sc"].view(np.float16).astype(np.float32)
    dead = (sc[:, 0::2] == 256.0) & (sc[:, 1::2] == -384.0)           # s <= 0 -> 1
    assert dead.any() and not dead.all()
    i = int(np.argmax(dead.all(1)))                                   # the all-zero row: every code 128
    assert np.all(gold["k_dw"][i] == 0x80808080)
    assert np.isinf(sc).any()                                         # 256 s beyond the f16 range
    st = gold["v_st"].view(np.float16).astype(np.float32)
    assert ((st[..., 0] == 256.0) & np.all(gold["v_dw"] == 0x80808080, -1)).any()   # a constant channel


def pools_from_chunk(rc, n_tokens, fill=0):
    g = kv8.geometry(24, 4, rc.T // 256)
    hp = kv8.HostPools(g, fill)
    hp.km[rc.ptab[0]] = rc.m
    kv8.append(hp, rc.ptab[None], [0], None, rc.K[None, :n_tokens].astype(np.float32),
               rc.V[None, :n_tokens].astype(np.float32))
    return hp


def test_recipe_pools_bit_exact(rc):
    g = rc.g
    full = pools_from_chunk(rc, rc.T)                    # the checker quantizes every K row of the pool
    assert np.array_equal(kv8_recipe.sha(full.kq), g["rc_kq_sha"])
    assert np.array_equal(full.ks.view(np.uint16).reshape(rc.T, 16), g["rc_ks"])
    assert np.array_equal(full.kq[g["rc_kq_rows_idx"]], g["rc_kq_rows"])
    assert np.array_equal(kv8_recipe.sha(kv8.dense(full, rc.ptab, rc.T)[0]), g["rc_Kd_sha"])
    hp = pools_from_chunk(rc, rc.n, fill=0x5A)           # ... and the V tiles before the newest
    closed = [kv8_recipe.ptile(rc, t) for t in range(rc.curt)]
    vq, vs = np.zeros_like(hp.vq), np.zeros_like(hp.vs)
    vq[:, closed], vs[:, closed] = hp.vq[:, closed], hp.vs[:, closed]
    assert np.array_equal(kv8_recipe.sha(vq), g["rc_vq_sha"])
    assert np.array_equal(vs.view(np.uint16).reshape(4, -1, 256, 2), g["rc_vs"])
    assert np.array_equal(vq[:, g["rc_vq_tiles_idx"]], g["rc_vq_tiles"])
    # the open tile: the keys so far, and (the chunk form) zeros after them
    vo = hp.vo[rc.ptab[rc.pos // 256]]
    assert np.array_equal(vo[:, :rc.nk], g["rc_vopen"][:, :rc.nk])
    assert np.all(vo[:, rc.nk:] == 0)
    # pages of other positions were not touched: rows past the chunk keep the fill
    untouched = [kv8_recipe.prow(rc, p) for p in range(rc.n, rc.T)]
    assert np.all(hp.kq[untouched] == 0x5A5A5A5A) and np.all(hp.ks[untouched] == 0x5A5A5A5A)
    later = [kv8_recipe.ptile(rc, t) for t in range(rc.curt + 1, rc.T // 16)]
    assert np.all(hp.vq[:, later] == 0x5A5A5A5A) and np.all(hp.vs[:, later] == 0x5A5A5A5A)


def test_recipe_dense_model_and_attention(rc):
    g = rc.g
    hp = pools_from_chunk(rc, rc.n)
    hp.vo[rc.ptab[rc.pos // 256]][:, rc.nk:] = np.float16(7.0).view(np.uint16)   # stale keys past pos: masked (:177)
    Kd, Vd = kv8.dense(hp, rc.ptab, rc.n)
    Vfull = rc.V.astype(np.float32).copy()
    Vfull[:rc.n] = Vd.reshape(rc.n, 1024)
    assert np.array_equal(kv8_recipe.sha(Vfull), g["rc_Vd_sha"])
    out = closed_form(Kd, Vd, rc.q, 1.0 / 16.0, rc.gate)
    assert rel_err(out, g["rc_ref"]) < 1e-12
    assert 1e-4 < rel_err(g["rc_ref"], g["rc_exact"]) < 5e-2     # what quantization itself costs, for scale


def test_recipe_kappend(rc):
    g = rc.g
    hp = pools_from_chunk(rc, rc.T)
    before = {n: a.copy() for n, a in hp.arrays().items()}
    p2 = int(g["rc_p2"])
    kv8.append(hp, rc.ptab[None], [p2], None, g["rc_kx"][None, None], np.zeros((1, 1, 1024), np.float32))
    r = kv8_recipe.prow(rc, p2)
    assert np.array_equal(hp.kq[r], g["rc_k2_dw"])
    assert np.array_equal(hp.ks[r].view(np.uint16), g["rc_k2_sc"])
    assert np.array_equal(np.delete(hp.kq, r, 0), np.delete(before["kq"], r, 0))
    assert np.array_equal(np.delete(hp.ks, r, 0), np.delete(before["ks"], r, 0))
    assert np.array_equal(hp.vq, before["vq"]) and np.array_equal(hp.vs, before["vs"])   # p2 % 16 != 15


@pytest.mark.parametrize("case", [0, 1])
def test_recipe_vappend_mid_tile_and_closing(rc, case):
    g = rc.g
    hp = pools_from_chunk(rc, rc.n)
    p3 = int(g[f"rc_p3_{case}"])
    page = int(rc.ptab[p3 // 256])
    hp.vo[page] = g[f"rc_vo_{case}"]
    before = {n: a.copy() for n, a in hp.arrays().items()}
    kv8.append(hp, rc.ptab[None], [p3], None, rc.K[None, p3:p3 + 1].astype(np.float32), g[f"rc_vx_{case}"][None, None])
    assert np.array_equal(hp.vo[page], g[f"rc_vo_out_{case}"])
    pt = kv8_recipe.ptile(rc, p3 // 16)
    if p3 % 16 == 15:
        assert np.array_equal(hp.vq[:, pt], g["rc_v3_dw"])
        assert np.array_equal(hp.vs[:, pt].view(np.uint16).reshape(4, 256, 2), g["rc_v3_st"])
    else:
        assert np.array_equal(hp.vq[:, pt], before["vq"][:, pt])
    assert np.array_equal(np.delete(hp.vq, pt, 1), np.delete(before["vq"], pt, 1))
    assert np.array_equal(np.delete(hp.vs, pt, 1), np.delete(before["vs"], pt, 1))


def test_token_by_token_equals_chunk_on_closed_tiles(rc):
    """The decoder's appends and the prefill's chunk leave the same codes: K rows, and every V tile that closed."""
    n = 100
    a, b = pools_from_chunk(rc, n), kv8.HostPools(kv8.geometry(24, 4, rc.T // 256))
    b.km[rc.ptab[0]] = rc.m
    for p in range(n):
        kv8.append(b, rc.ptab[None], [p], None, rc.K[None, p:p + 1].astype(np.float32), rc.V[None, p:p + 1].astype(np.float32))
    rows = [kv8_recipe.prow(rc, p) for p in range(n)]
    assert np.array_equal(a.kq[rows], b.kq[rows]) and np.array_equal(a.ks[rows], b.ks[rows])
    closed = [kv8_recipe.ptile(rc, t) for t in range(n // 16)]
    assert np.array_equal(a.vq[:, closed], b.vq[:, closed]) and np.array_equal(a.vs[:, closed], b.vs[:, closed])
    page = int(rc.ptab[0])
    assert np.array_equal(a.vo[page][:, :n % 16], b.vo[page][:, :n % 16])
    # a chunk that starts inside a tile picks the tile's earlier keys up from the open tile
    c = pools_from_chunk(rc, 37)
    kv8.append(c, rc.ptab[None], [37], None, rc.K[None, 37:n].astype(np.float32), rc.V[None, 37:n].astype(np.float32))
    for name in ("kq", "ks", "vq", "vs"):
        assert np.array_equal(getattr(a, name), getattr(c, name)), name
    assert np.array_equal(a.vo[page][:, :n % 16], c.vo[page][:, :n % 16])


def test_kmean_order_and_value():
    rng = np.random.default_rng(9)
    k = (rng.standard_normal((333, 512)) * 3 + rng.standard_normal(512)).astype(np.float32)
    m = kv8.kmean(k)
    k16 = k.astype(np.float16).astype(np.float32)
    want = k16.astype(np.float64).mean(0)
    assert np.abs(m - want).max() < 333 * 2.0 ** -24 * np.abs(k16).max()
    # the order of sums: eight row groups, each in row order, then the groups in order
    grp = np.zeros((8, 512), np.float32)
    for r in range(333):
        grp[r % 8] = grp[r % 8] + k16[r]
    tot = np.zeros(512, np.float32)
    for gi in range(8):
        tot = tot + grp[gi]
    assert np.array_equal(m, tot / np.float32(333))


def test_prefill_side_decode_is_the_rounded_exact_value(rc):
    hp = pools_from_chunk(rc, 200)
    Kd, Vd = kv8.dense(hp, rc.ptab, 192)                 # (a length on a tile boundary's far side: all tiles closed but one)
    Kh, Vh = kv8.dense(hp, rc.ptab, 192, as_f16=True)
    assert np.array_equal(Kh, Kh.astype(np.float16).astype(np.float32))
    # exact value f * S + C' in float64, rounded once
    rows = [kv8_recipe.prow(rc, p) for p in range(192)]
    u = hp.kq[rows].view(np.uint8).reshape(192, 256, 4)[:, :, [0, 2, 1, 3]].reshape(192, 8, 128).astype(np.float64)
    sc = hp.ks[rows].view(np.float16).reshape(192, 8, 2).astype(np.float64)
    exact = (1 + u / 256) * sc[:, :, :1] + sc[:, :, 1:]
    assert np.array_equal(Kh.reshape(192, 8, 128), exact.astype(np.float16).astype(np.float32))
    # against the decode side's f32 form: C' = f16(-384 s) is off by up to 2^-11 * 384 s = 0.19 steps, and the product rounds
    assert np.abs(Kh - Kd).max() <= 0.5 * np.abs(Kd).max() / 127
    closed = 192 // 16 - 1
    assert np.abs(Vh[:16 * closed] - Vd[:16 * closed]).max() <= 0.5 * 2 * np.abs(Vd).max() / 254
