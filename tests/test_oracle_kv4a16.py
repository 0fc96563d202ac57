"""The CPU oracle of the reference's 4-bit KV format, kv4a16 (oracle/kv8_oracle.c, orc_kv4_*), against the reference's
numpy model of it: tests/golden/kv4a16_vectors.npz holds inputs and outputs of quant_k, deq_k, quant_vtile, deq_vtile
with bits = 4 (engine/gpu/loom/tools/dattn_q_check.py:52-137) and of the checker's whole recipe (:140-256).

The model rotates K in float64; the reference's kernel and the oracle run the butterflies in f32 in a fixed order. The
"exact" rows are built so that every partial sum is exact: there the oracle must agree bit for bit. On random rows a
rotated value may differ in its last bit, which moves a code by one step where the value sits on a rounding boundary
and a scale by one f16 step: the reference's own checker accepts exactly that (`codes exact or differ`, dequantized
values within 1e-2, dattn_q_check.py:222-225)."""
import numpy as np
import pytest

import kv8_recipe
from helpers import closed_form, rel_err
from oracle import kv8


@pytest.fixture(scope="module")
def gold():
    return kv8_recipe.golden(4)


@pytest.fixture(scope="module")
def rc():
    return kv8_recipe.load(4)


def nibbles(dw):
    """K code dwords [..., n] -> codes [..., 8 n] in dim order"""
    dw = np.asarray(dw, np.uint32)
    sh = np.array([4 * (i // 2) + (16 if i % 2 else 0) for i in range(8)], np.uint32)
    return ((dw[..., None] >> sh) & 15).reshape(*dw.shape[:-1], -1).astype(np.int32)


def test_hadamard_is_the_matrix(gold):
    """Sign and index order of the butterfly: unit vectors give columns of H, random vectors H x to f32 accuracy."""
    got = kv8.hadamard256(gold["had_in"])
    want = gold["had_out"]
    assert np.array_equal(got[:2].astype(np.float64), want[:2])              # the two unit vectors: +-1 exactly
    assert np.abs(got - want).max() < 256 * 2.0 ** -22 * np.abs(gold["had_in"]).max()
    assert np.array_equal(kv8.rotate_q(gold["had_in"][:2]).astype(np.float64), want[:2] / 16)


def test_exact_k_rows_bit_exact(gold):
    zero = np.zeros(1024, np.float32)
    for i in range(gold["kx_in"].shape[0]):
        dw, sc = kv8.quant_k4(gold["kx_in"][i], zero)
        assert np.array_equal(dw, gold["kx_dw"][i]), f"K row {i}: codes"
        assert np.array_equal(sc, gold["kx_sc"][i]), f"K row {i}: scale pairs"
        assert np.array_equal(kv8.deq_k4(gold["kx_dw"][i], gold["kx_sc"][i]).view(np.uint32),
                              gold["kx_deq"][i].view(np.uint32)), f"K row {i}: dequantized values"


def test_exact_rows_say_what_they_should(gold):
    sc = gold["kx_sc"].view(np.float16).astype(np.float32).reshape(-1, 32, 2)
    u = nibbles(gold["kx_dw"]).reshape(-1, 32, 32)
    assert np.array_equal(u[0, 0, :10], [0, 15, 0, 2, 2, 4, 14, 14, 8, 8])     # ties go to the even code
    assert sc[0, 0, 0] == 16.0 and sc[0, 0, 1] == -16.0                         # s = 1: (16 s, lo - 16 s)
    dead = (sc[..., 0] == 16.0) & np.all(u == 0, -1)                            # s0 = 0 -> s = 1, every code 0
    assert dead.any() and not dead.all()
    assert (sc[..., 1] + sc[..., 0] < 0).any()                                  # negative lows
    assert set(np.unique(u)) == set(range(16))


def test_random_k_rows_within_the_rotation_rounding(gold):
    n_codes = n_diff = 0
    for i in range(gold["kr_in"].shape[0]):
        dw, sc = kv8.quant_k4(gold["kr_in"][i], gold["kr_mean"][i])
        a, b = nibbles(dw), nibbles(gold["kr_dw"][i])
        assert np.abs(a - b).max() <= 1, f"K row {i}"
        n_codes += a.size
        n_diff += int((a != b).sum())
        mine, theirs = kv8.deq_k4(dw, sc), gold["kr_deq"][i]
        step = np.abs(theirs).max() / 7
        assert np.abs(mine - theirs).max() <= 1.01 * step, f"K row {i}"         # at most the step of a moved code
        s1, s2 = sc.view(np.float16).astype(np.float32), gold["kr_sc"][i].view(np.float16).astype(np.float32)
        assert np.all(np.abs(s1 - s2) <= 2.0 ** -10 * np.abs(s2) + 1e-12), f"K row {i}: scales"   # one f16 step
    assert n_diff <= 2e-3 * n_codes, (n_diff, n_codes)


def test_v_tiles_bit_exact(gold):
    for i in range(gold["v_in"].shape[0]):
        dw, st = kv8.quant_vtile4(gold["v_in"][i])
        assert np.array_equal(dw, gold["v_dw"][i]), f"V tile {i}: codes"
        assert np.array_equal(st, gold["v_st"][i]), f"V tile {i}: stats"
        assert np.array_equal(kv8.deq_vtile4(gold["v_dw"][i], gold["v_st"][i]).view(np.uint32),
                              gold["v_deq"][i].view(np.uint32)), f"V tile {i}: dequantized values"
    assert int((gold["v_dw"] & 15).max()) == 14 and int(((gold["v_dw"] >> 28) & 15).max()) == 14   # 15 levels


def pools_from_chunk(rc, n_tokens, fill=0, k_bits=4, v_bits=4):
    g = kv8.geometry(24, 4, rc.T // 256, k_bits, v_bits)
    hp = kv8.HostPools(g, fill)
    hp.km[rc.ptab[0]] = rc.m
    kv8.append(hp, rc.ptab[None], [0], None, rc.K[None, :n_tokens].astype(np.float32),
               rc.V[None, :n_tokens].astype(np.float32))
    return hp


def test_recipe_pools(rc):
    g = rc.g
    full = pools_from_chunk(rc, rc.T)
    a, b = nibbles(full.kq), nibbles(g["rc_kq"])
    assert np.abs(a - b).max() <= 1 and (a != b).mean() < 2e-3                # K: within the rotation's rounding
    s1 = full.ks.view(np.float16).astype(np.float32).reshape(rc.T, 64)
    s2 = g["rc_ks"].view(np.float16).astype(np.float32)
    assert np.all(np.abs(s1 - s2) <= 2.0 ** -10 * np.abs(s2)) and (s1 != s2).mean() < 2e-3
    hp = pools_from_chunk(rc, rc.n, fill=0x5A)                                # V: bit for bit
    closed = [kv8_recipe.ptile(rc, t) for t in range(rc.curt)]
    vq, vs = np.zeros_like(hp.vq), np.zeros_like(hp.vs)
    vq[:, closed], vs[:, closed] = hp.vq[:, closed], hp.vs[:, closed]
    assert np.array_equal(kv8_recipe.sha(vq), g["rc_vq_sha"])
    assert np.array_equal(vs.view(np.uint16).reshape(4, -1, 256, 2), g["rc_vs"])
    assert np.array_equal(vq[:, g["rc_vq_tiles_idx"]], g["rc_vq_tiles"])
    vo = hp.vo[rc.ptab[rc.pos // 256]]
    assert np.array_equal(vo[:, :rc.nk], g["rc_vopen"][:, :rc.nk]) and np.all(vo[:, rc.nk:] == 0)
    untouched = [kv8_recipe.prow(rc, p) for p in range(rc.n, rc.T)]
    assert np.all(hp.kq[untouched] == 0x5A5A5A5A) and np.all(hp.ks[untouched] == 0x5A5A5A5A)
    later = [kv8_recipe.ptile(rc, t) for t in range(rc.curt + 1, rc.T // 16)]
    assert np.all(hp.vq[:, later] == 0x5A5A5A5A) and np.all(hp.vs[:, later] == 0x5A5A5A5A)


def test_recipe_dense_model_and_attention(rc):
    g = rc.g
    hp = pools_from_chunk(rc, rc.n)
    hp.vo[rc.ptab[rc.pos // 256]][:, rc.nk:] = np.float16(7.0).view(np.uint16)
    Kd, Vd = kv8.dense(hp, rc.ptab, rc.n)
    Vfull = rc.V.astype(np.float32).copy()
    Vfull[:rc.n] = Vd.reshape(rc.n, 1024)
    assert np.array_equal(kv8_recipe.sha(Vfull), g["rc_Vd_sha"])
    qr = kv8.rotate_q(rc.q)
    assert np.abs(qr - g["rc_qr"]).max() < 1e-6
    out = closed_form(Kd, Vd, qr, 1.0 / 16.0, rc.gate)
    assert rel_err(out, g["rc_ref"]) < 3e-4          # the few K codes that moved by a step
    assert 1e-3 < rel_err(g["rc_ref"], g["rc_exact"]) < 0.3      # what 4-bit quantization itself costs, for scale
    # the rotation leaves the scores alone: unrotated q against the inverse-rotated K gives the same attention
    Kn = kv8.hadamard256(Kd.reshape(rc.n, 4, 256)) / 16
    assert rel_err(closed_form(Kn, Vd, rc.q, 1.0 / 16.0, rc.gate), out) < 1e-5


def test_recipe_kappend(rc):
    g = rc.g
    hp = pools_from_chunk(rc, rc.T)
    before = {n: a.copy() for n, a in hp.arrays().items()}
    p2 = int(g["rc_p2"])
    kv8.append(hp, rc.ptab[None], [p2], None, g["rc_kx"][None, None], np.zeros((1, 1, 1024), np.float32))
    r = kv8_recipe.prow(rc, p2)
    assert np.abs(nibbles(hp.kq[r]) - nibbles(g["rc_k2_dw"])).max() <= 1
    assert np.abs(kv8.deq_k4(hp.kq[r], hp.ks[r].view(np.uint16)) - kv8.deq_k4(g["rc_k2_dw"], g["rc_k2_sc"])).max() < 1e-2
    dw, sc = kv8.quant_k4(g["rc_kx"], rc.m)
    assert np.array_equal(hp.kq[r], dw) and np.array_equal(hp.ks[r].view(np.uint16), sc)
    assert np.array_equal(np.delete(hp.kq, r, 0), np.delete(before["kq"], r, 0))
    assert np.array_equal(np.delete(hp.ks, r, 0), np.delete(before["ks"], r, 0))
    assert np.array_equal(hp.vq, before["vq"]) and np.array_equal(hp.vs, before["vs"])


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
    n = 100
    a, b = pools_from_chunk(rc, n), kv8.HostPools(kv8.geometry(24, 4, rc.T // 256, 4, 4))
    b.km[rc.ptab[0]] = rc.m
    for p in range(n):
        kv8.append(b, rc.ptab[None], [p], None, rc.K[None, p:p + 1].astype(np.float32), rc.V[None, p:p + 1].astype(np.float32))
    rows = [kv8_recipe.prow(rc, p) for p in range(n)]
    assert np.array_equal(a.kq[rows], b.kq[rows]) and np.array_equal(a.ks[rows], b.ks[rows])
    closed = [kv8_recipe.ptile(rc, t) for t in range(n // 16)]
    assert np.array_equal(a.vq[:, closed], b.vq[:, closed]) and np.array_equal(a.vs[:, closed], b.vs[:, closed])


@pytest.mark.parametrize("kb,vb", [(8, 4), (4, 8)])
def test_mixed_formats_take_each_side_from_its_own_codec(rc, kb, vb):
    """k8v4 / k4v8 (the reference's `kv q KB VB`): K as the KB-bit format alone would store it, V as the VB-bit one."""
    mixed = pools_from_chunk(rc, 300, k_bits=kb, v_bits=vb)
    kside, vside = pools_from_chunk(rc, 300, k_bits=kb, v_bits=kb), pools_from_chunk(rc, 300, k_bits=vb, v_bits=vb)
    assert np.array_equal(mixed.kq, kside.kq) and np.array_equal(mixed.ks, kside.ks)
    assert np.array_equal(mixed.vq, vside.vq) and np.array_equal(mixed.vs, vside.vs)


def test_prefill_side_decode_is_the_rounded_exact_value(rc):
    hp = pools_from_chunk(rc, 200)
    Kd, Vd = kv8.dense(hp, rc.ptab, 192)
    Kh, Vh = kv8.dense(hp, rc.ptab, 192, as_f16=True)
    assert np.array_equal(Kh, Kh.astype(np.float16).astype(np.float32))
    rows = [kv8_recipe.prow(rc, p) for p in range(192)]
    u = nibbles(hp.kq[rows]).reshape(192, 32, 32).astype(np.float64)
    sc = hp.ks[rows].view(np.float16).reshape(192, 32, 2).astype(np.float64)
    exact = (1 + u / 16) * sc[:, :, :1] + sc[:, :, 1:]
    assert np.array_equal(Kh.reshape(192, 32, 32), exact.astype(np.float16).astype(np.float32))
    assert np.abs(Kh - Kd).max() <= 2.0 ** -10 * np.abs(Kd).max()
    closed = 192 // 16 - 1
    assert np.abs(Vh[:16 * closed] - Vd[:16 * closed]).max() <= 2.0 ** -10 * np.abs(Vd).max()
