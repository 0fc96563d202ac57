"""The CPU oracle's page scatter and attention against an independent numpy reading of the layout, the float64
closed form and the special cases that a dropped term, a wrong index or a transposed operand would break."""
import numpy as np
import pytest

import oracle
from helpers import closed_form, dequant, logical_blocks, make_tables, rel_err, to_f16_f32


def build(fmt, n_q, n_kv, hd, pt, lens, seed, extra_pages=0, poison=0xA5):
    rng = np.random.default_rng(seed)
    pages = [(n + pt - 1) // pt for n in lens]
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, sum(pages) + extra_pages)
    table = make_tables(rng, pages, g.n_pages)
    pools = oracle.HostPools(g, fill=poison)
    K = [to_f16_f32(rng.standard_normal((n, n_kv, hd))) for n in lens]
    V = [to_f16_f32(rng.standard_normal((n, n_kv, hd))) for n in lens]
    for s, n in enumerate(lens):                                    # each sequence appended as one chunk
        oracle.append(pools, table[s:s + 1], [0], None, K[s][None], V[s][None])
    return g, table, pools, K, V, rng


@pytest.mark.parametrize("fmt", [8, 4])
def test_append_gather_equals_contiguous_quantize(fmt):
    g, table, pools, K, V, _ = build(fmt, 8, 2, 128, 16, [40, 7, 33], seed=1, extra_pages=3)
    quant = oracle.quantize_q8_0 if fmt == 8 else oracle.quantize_q4_0
    bb = 34 if fmt == 8 else 18
    for s, n in enumerate([40, 7, 33]):
        k, v = oracle.gather_blocks(pools, table[s], n)
        assert np.array_equal(k.reshape(-1, bb), quant(K[s]))
        assert np.array_equal(v.reshape(-1, bb), quant(V[s]))
        # the documented layout read with numpy indexing gives the same blocks
        (ks, kc), (vs, vc) = logical_blocks(pools.arrays(), g, table[s], n)
        assert np.array_equal(ks.reshape(-1), k.reshape(-1, bb)[:, :2].copy().view(np.uint16).reshape(-1))
        deq = oracle.dequantize_q8_0 if fmt == 8 else oracle.dequantize_q4_0
        assert np.array_equal(dequant(ks, kc).reshape(-1), deq(k))
        assert np.array_equal(dequant(vs, vc).reshape(-1), deq(v))


@pytest.mark.parametrize("fmt", [8, 4])
def test_append_touches_only_its_slots(fmt):
    g, table, pools, K, V, rng = build(fmt, 8, 2, 128, 16, [20], seed=2, extra_pages=2, poison=0x5A)
    before = {k: v.copy() for k, v in pools.arrays().items()}
    # one more token at position 20 -> page table[0][1], slot 4
    oracle.append(pools, table, [20], None, rng.standard_normal((1, 1, 2, 128)), rng.standard_normal((1, 1, 2, 128)))
    H, D, PT, NB, P = 2, 128, 16, 4, g.n_pages
    page, t = table[0, 1], 4
    cb = 32 if fmt == 8 else 16
    masks = {"kq": np.zeros((P, H, NB, PT, cb), bool), "ks": np.zeros((P, H, PT, NB), bool),
             "vs": np.zeros((P, H, NB, PT), bool)}
    masks["kq"][page, :, :, t, :] = True
    masks["ks"][page, :, t, :] = True
    masks["vs"][page, :, :, t] = True
    if fmt == 8:
        masks["vq"] = np.zeros((P, H, D, PT), bool)
        masks["vq"][page, :, :, t] = True
    else:
        masks["vq"] = np.zeros((P, H, NB, 16, PT), bool)
        masks["vq"][page, :, :, :, t] = True
    for name, arr in pools.arrays().items():
        m = masks[name].reshape(-1)
        assert np.array_equal(arr[~m], before[name][~m]), name       # every other byte untouched
    # unused pages still hold the poison
    unused = sorted(set(range(P)) - set(table[0, :2].tolist()))
    assert np.all(pools.kq.reshape(P, -1)[unused] == 0x5A)


def test_append_n_valid_and_token_by_token_equals_chunk():
    rng = np.random.default_rng(3)
    g = oracle.geometry(8, 8, 2, 128, 16, 6)
    table = make_tables(rng, [3, 3], 6)
    K = to_f16_f32(rng.standard_normal((2, 40, 2, 128)))
    V = to_f16_f32(rng.standard_normal((2, 40, 2, 128)))
    a, b = oracle.HostPools(g, fill=1), oracle.HostPools(g, fill=1)
    oracle.append(a, table, [0, 0], [40, 23], K, V)                      # padded chunk: sequence 1 has 23 real rows
    for t in range(40):
        oracle.append(b, table[:1], [t], None, K[:1, t:t + 1], V[:1, t:t + 1])
    for t in range(23):
        oracle.append(b, table[1:], [t], None, K[1:, t:t + 1], V[1:, t:t + 1])
    for name in ("kq", "ks", "vq", "vs"):
        assert np.array_equal(a.arrays()[name], b.arrays()[name]), name


def attend_all(g, table, pools, lens, q, scale, gate=None):
    want = np.zeros(q.shape)
    for s, n in enumerate(lens):
        (ks, kc), (vs, vc) = logical_blocks(pools.arrays(), g, table[s], n)
        want[s] = closed_form(dequant(ks, kc), dequant(vs, vc), q[s], scale, None if gate is None else gate[s])
    return want


def test_decode_config1_tiny_against_closed_form():
    """Configuration 1: 1 sequence, 8 Q / 2 KV heads, head_dim 128, 16-token pages, 512-token prefix + 1 appended."""
    rng = np.random.default_rng(1)
    g = oracle.geometry(8, 8, 2, 128, 16, 33)
    K = to_f16_f32(rng.standard_normal((1, 513, 2, 128)))
    V = to_f16_f32(rng.standard_normal((1, 513, 2, 128)))
    table = np.random.default_rng(2).permutation(33).astype(np.int32)[None]
    q = to_f16_f32(np.random.default_rng(3).standard_normal((1, 8, 128)))
    pools = oracle.HostPools(g, fill=0x77)
    oracle.append(pools, table, [0], None, K[:, :512], V[:, :512])
    oracle.append(pools, table, [512], None, K[:, 512:], V[:, 512:])
    scale = 1 / np.sqrt(128)
    got = oracle.decode_attend(pools, table, [513], q, scale)
    want = attend_all(g, table, pools, [513], q, scale)
    assert rel_err(got, want) < 2e-6
    # the appended token is visible in this step and not in the one before (key < pos + 1)
    prev = oracle.decode_attend(pools, table, [512], q, scale)
    assert rel_err(prev, attend_all(g, table, pools, [512], q, scale)) < 2e-6
    assert np.abs(prev - got).max() > 1e-6
    # quantization error vs unquantized fp16 K/V, reported by the reference checker as well (dattn_q_check.py:204)
    exact = closed_form(K[0], V[0], q[0], scale)
    assert rel_err(got[0], exact) < 2e-2


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt", [(8, 24, 4, 256, 64), (4, 24, 4, 256, 64), (8, 8, 2, 128, 16), (4, 6, 1, 128, 32)])
def test_decode_ragged_batch_with_gate(fmt, n_q, n_kv, hd, pt):
    lens = [1, pt - 1, pt, pt + 1, 3 * pt + 5, 200]
    g, table, pools, K, V, rng = build(fmt, n_q, n_kv, hd, pt, lens, seed=4, extra_pages=2)
    q = 0.3 * rng.standard_normal((len(lens), n_q, hd)).astype(np.float32)
    gate = rng.standard_normal((len(lens), n_q, hd)).astype(np.float32)
    scale = 1 / np.sqrt(hd)
    got = oracle.decode_attend(pools, table, lens, q, scale, gate)
    assert rel_err(got, attend_all(g, table, pools, lens, q, scale, gate)) < 3e-6
    nog = oracle.decode_attend(pools, table, lens, q, scale)
    assert rel_err(nog, attend_all(g, table, pools, lens, q, scale)) < 3e-6
    assert np.allclose(got, nog / (1 + np.exp(-gate.astype(np.float64))), rtol=1e-5, atol=1e-7)


def test_decode_special_cases():
    g, table, pools, K, V, rng = build(8, 8, 2, 128, 16, [1, 50], seed=5)
    (ks, kc), (vs, vc) = logical_blocks(pools.arrays(), g, table[0], 1)
    Vd0 = dequant(vs, vc)[0]                                          # [H][D]
    q = rng.standard_normal((2, 8, 128)).astype(np.float32)
    out = oracle.decode_attend(pools, table, [1, 50], q, 0.1)
    assert np.array_equal(out[0], np.repeat(Vd0, 4, 0))               # one key: out == its dequantized V, exactly
    # q = 0: all scores equal -> the mean of V
    out = oracle.decode_attend(pools, table, [1, 50], np.zeros_like(q), 0.1)
    (_, _), (vs, vc) = logical_blocks(pools.arrays(), g, table[1], 50)
    assert np.allclose(out[1], np.repeat(dequant(vs, vc).mean(0), 4, 0), rtol=1e-5, atol=1e-6)
    # heads of one GQA group with equal queries give equal outputs
    q[1, 1] = q[1, 0]
    out = oracle.decode_attend(pools, table, [1, 50], q, 0.1)
    assert np.array_equal(out[1, 0], out[1, 1]) and not np.array_equal(out[1, 0], out[1, 4])
    # one enormous score: that key's V row
    (ks, kc), (vs, vc) = logical_blocks(pools.arrays(), g, table[1], 50)
    Kd, Vd = dequant(ks, kc), dequant(vs, vc)
    q[1, 5] = 50 * Kd[17, 1] / np.linalg.norm(Kd[17, 1])
    out = oracle.decode_attend(pools, table, [1, 50], q, 1.0)
    assert np.allclose(out[1, 5], Vd[17, 1], atol=1e-5)
    # length 0: zeros
    out = oracle.decode_attend(pools, table, [0, 50], q, 0.1)
    assert np.all(out[0] == 0)


def test_decode_invariant_under_page_permutation():
    """Moving pages (table and pool contents together) leaves the output bit-identical: the merge is by logical page."""
    g, table, pools, K, V, rng = build(8, 8, 2, 128, 16, [100, 37], seed=6, extra_pages=4)
    q = rng.standard_normal((2, 8, 128)).astype(np.float32)
    a = oracle.decode_attend(pools, table, [100, 37], q, 0.09)
    perm = rng.permutation(g.n_pages)                                  # new physical id of old page i
    moved = oracle.HostPools(g)
    for name, arr in pools.arrays().items():
        dst = moved.arrays()[name].reshape(g.n_pages, -1)
        dst[perm] = arr.reshape(g.n_pages, -1)
    b = oracle.decode_attend(moved, perm[table].astype(np.int32), [100, 37], q, 0.09)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("fmt", [8, 4])
def test_prefill_against_closed_form_and_decode(fmt):
    pt, hd, n_q, n_kv = 16, 128, 8, 2
    prefix, chunk = [37, 0, 64], 21
    lens = [p + chunk for p in prefix]
    g, table, pools, K, V, rng = build(fmt, n_q, n_kv, hd, pt, lens, seed=7, extra_pages=1)
    q = 0.5 * rng.standard_normal((3, chunk, n_q, hd)).astype(np.float32)
    gate = rng.standard_normal((3, chunk, n_q, hd)).astype(np.float32)
    scale = 1 / np.sqrt(hd)
    got = oracle.prefill_attend(pools, table, prefix, q, scale, gate)
    for s in range(3):
        (ks, kc), (vs, vc) = logical_blocks(pools.arrays(), g, table[s], lens[s])
        Kd, Vd = dequant(ks, kc), dequant(vs, vc)
        for t in (0, 1, chunk // 2, chunk - 1):
            n = prefix[s] + t + 1                                       # causal: keys 0 .. prefix + t
            want = closed_form(Kd[:n], Vd[:n], q[s, t], scale, gate[s, t])
            assert rel_err(got[s, t], want) < 1e-6
    # a chunk of one query equals decode attention at that length
    one = oracle.prefill_attend(pools, table, [l - 1 for l in lens], q[:, -1:], scale, gate[:, -1:])
    dec = oracle.decode_attend(pools, table, lens, q[:, -1], scale, gate[:, -1])
    assert rel_err(one[:, 0], dec) < 3e-6
