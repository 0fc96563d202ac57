"""kv8a16, the reference's own KV format, on the GPU through the C ABI (yahkv_kv8_*): pools bit for bit against the
fixtures written from the reference's numpy model (tests/golden/kv8a16_vectors.npz, dattn_q_check.py:61-256) and
against the CPU oracle restating it; attention against the float64 closed form over the dequantized model, held to 2e-3
and reported against the reference checker's own 1e-4 (dattn_q_check.py:205-208)."""
import numpy as np
import pytest

import kv8_recipe
from helpers import closed_form, rel_err
from oracle import kv8

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.fixture(scope="module")
def rc():
    return kv8_recipe.load()


def dev_pools(yahkv, torch, rc, n_tokens, fill=0):
    g = yahkv.kv8_geometry(24, 4, rc.T // 256)
    dp = yahkv.Kv8Pools(g, fill)
    arrs = dp.numpy()
    arrs["km"][rc.ptab[0]] = rc.m
    dp.load(arrs)
    table = torch.from_numpy(rc.ptab[None].copy()).cuda()
    if n_tokens:
        yahkv.kv8_append(dp, table, torch.zeros(1, dtype=torch.int32, device="cuda"),
                         torch.from_numpy(rc.K[None, :n_tokens].reshape(1, n_tokens, 4, 256)).cuda(),
                         torch.from_numpy(rc.V[None, :n_tokens].reshape(1, n_tokens, 4, 256)).cuda())
    return dp, table


def host_pools(rc, n_tokens, fill=0):
    hp = kv8.HostPools(kv8.geometry(24, 4, rc.T // 256), fill)
    hp.km[rc.ptab[0]] = rc.m
    if n_tokens:
        kv8.append(hp, rc.ptab[None], [0], None, rc.K[None, :n_tokens].astype(np.float32), rc.V[None, :n_tokens].astype(np.float32))
    return hp


def same(got, want, what):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, f"{what}: shape {got.shape} against {want.shape}"
    bad = np.argwhere(got != want)
    assert bad.size == 0, (f"{what}: {len(bad)} of {got.size} differ, first at {bad[:6].tolist()}: got "
                           f"{[hex(int(got[tuple(b)])) for b in bad[:6]]} want {[hex(int(want[tuple(b)])) for b in bad[:6]]}")


def assert_pools_equal(dp, hp, what=""):
    got = dp.numpy()
    for name, want in hp.arrays().items():
        if name == "km":
            assert np.array_equal(got[name].view(np.uint32), want.view(np.uint32)), f"{what}: km"
        else:
            bad = np.argwhere(got[name] != want)
            assert bad.size == 0, f"{what}: {name} differs from the oracle at {bad[:4].tolist()} ({len(bad)} places)"


def test_recipe_chunk_append_bit_exact(yahkv, torch_gpu, rc):
    """The checker's pools (dattn_q_check.py:153-177) from one chunk append, against the fixture and the oracle, with
    every other byte of the poison-filled pools untouched."""
    g = rc.g
    dp, _ = dev_pools(yahkv, torch_gpu, rc, rc.n, fill=0x5A)
    torch_gpu.cuda.synchronize()
    got = dp.numpy()
    rows = np.array([kv8_recipe.prow(rc, p) for p in range(rc.n)])
    same(got["ks"][rows].view(np.uint16).reshape(rc.n, 16), g["rc_ks"][rows], "ks against the fixture")
    closed = [kv8_recipe.ptile(rc, t) for t in range(rc.curt)]
    same(got["vs"][:, closed].view(np.uint16).reshape(4, len(closed), 256, 2), g["rc_vs"][:, closed], "vs against the fixture")
    vq = np.zeros_like(got["vq"])
    vq[:, closed] = got["vq"][:, closed]
    assert np.array_equal(kv8_recipe.sha(vq), g["rc_vq_sha"])
    idx = [i for i, r in enumerate(g["rc_kq_rows_idx"]) if r in set(rows.tolist())]
    assert len(idx) > 10 and np.array_equal(got["kq"][g["rc_kq_rows_idx"][idx]], g["rc_kq_rows"][idx])
    assert np.array_equal(got["vo"][rc.ptab[rc.pos // 256]][:, :rc.nk], g["rc_vopen"][:, :rc.nk])
    assert_pools_equal(dp, host_pools(rc, rc.n, fill=0x5A), "chunk of 701")
    dp_full, _ = dev_pools(yahkv, torch_gpu, rc, rc.T)
    assert np.array_equal(kv8_recipe.sha(dp_full.numpy()["kq"]), g["rc_kq_sha"])      # every K row of the checker's pool


def test_recipe_kappend_and_vappend(yahkv, torch_gpu, rc):
    """dattn_q_check.py:210-250: the K append at position 517; the V append mid-tile and on the tile's 16th key."""
    torch, g = torch_gpu, rc.g
    dp, table = dev_pools(yahkv, torch, rc, rc.n, fill=0x33)
    hp = host_pools(rc, rc.n, fill=0x33)
    p2 = int(g["rc_p2"])
    kx = torch.from_numpy(g["rc_kx"].reshape(1, 1, 4, 256)).cuda()
    yahkv.kv8_append(dp, table, torch.tensor([p2], dtype=torch.int32, device="cuda"), kx, torch.zeros_like(kx))
    got = dp.numpy()
    r = kv8_recipe.prow(rc, p2)
    assert np.array_equal(got["kq"][r], g["rc_k2_dw"]) and np.array_equal(got["ks"][r].view(np.uint16), g["rc_k2_sc"])
    kv8.append(hp, rc.ptab[None], [p2], None, g["rc_kx"][None, None], np.zeros((1, 1, 1024), np.float32))
    assert_pools_equal(dp, hp, "kappend")
    for case in (0, 1):
        p3 = int(g[f"rc_p3_{case}"])
        page = int(rc.ptab[p3 // 256])
        arrs = dp.numpy()
        arrs["vo"][page] = g[f"rc_vo_{case}"]
        dp.load(arrs)
        hp.vo[page] = g[f"rc_vo_{case}"]
        vx = torch.from_numpy(g[f"rc_vx_{case}"].reshape(1, 1, 4, 256)).cuda()
        kk = torch.from_numpy(rc.K[p3].astype(np.float32).reshape(1, 1, 4, 256)).cuda()
        yahkv.kv8_append(dp, table, torch.tensor([p3], dtype=torch.int32, device="cuda"), kk, vx)
        got = dp.numpy()
        assert np.array_equal(got["vo"][page], g[f"rc_vo_out_{case}"]), f"vappend at {p3}: open tile"
        pt = kv8_recipe.ptile(rc, p3 // 16)
        if p3 % 16 == 15:
            assert np.array_equal(got["vq"][:, pt], g["rc_v3_dw"]), "closing key: codes"
            assert np.array_equal(got["vs"][:, pt].view(np.uint16).reshape(4, 256, 2), g["rc_v3_st"]), "closing key: stats"
        kv8.append(hp, rc.ptab[None], [p3], None, rc.K[None, p3:p3 + 1].astype(np.float32), g[f"rc_vx_{case}"][None, None])
        assert_pools_equal(dp, hp, f"vappend at {p3}")


def test_directed_rows_and_tiles_through_the_kernels(yahkv, torch_gpu):
    """The fixture's directed K rows (dead halves, ties, scales beyond f16) and V tiles through the append kernels."""
    torch = torch_gpu
    gold = kv8_recipe.golden()
    n = gold["k_in"].shape[0]
    g = yahkv.kv8_geometry(24, 4, n)                       # one sequence (one page) per row: each has its own means
    dp = yahkv.Kv8Pools(g)
    arrs = dp.numpy()
    arrs["km"][:] = gold["k_mean"]
    dp.load(arrs)
    table = torch.arange(n, dtype=torch.int32, device="cuda").reshape(n, 1)
    k = torch.from_numpy(gold["k_in"].reshape(n, 1, 4, 256)).cuda()
    yahkv.kv8_append(dp, table, torch.zeros(n, dtype=torch.int32, device="cuda"), k, torch.zeros_like(k))
    got = dp.numpy()
    for i in range(n):
        assert np.array_equal(got["kq"][i * 256], gold["k_dw"][i]), f"K row {i}: codes (one-token kernel)"
        assert np.array_equal(got["ks"][i * 256].view(np.uint16), gold["k_sc"][i]), f"K row {i}: scales"
    k2 = torch.cat([k, k], 1)                              # the chunk kernel: the same row twice
    yahkv.kv8_append(dp, table, torch.zeros(n, dtype=torch.int32, device="cuda"), k2, torch.zeros_like(k2))
    got = dp.numpy()
    for i in range(n):
        assert np.array_equal(got["kq"][i * 256 + 1], gold["k_dw"][i]), f"K row {i}: codes (chunk kernel)"
        assert np.array_equal(got["ks"][i * 256 + 1].view(np.uint16), gold["k_sc"][i])
    # V: sixteen 64-channel tiles side by side make one 1024-channel tile
    nt = gold["v_in"].shape[0]
    groups = [list(range(i, min(i + 16, nt))) + [0] * max(0, i + 16 - nt) for i in range(0, nt, 16)]
    v = np.stack([np.concatenate([gold["v_in"][j] for j in grp], 1) for grp in groups])       # [seq][16][1024] f16 bits
    vt = torch.from_numpy(v.view(np.float16).reshape(len(groups), 16, 4, 256).copy()).cuda()
    table2 = table[:len(groups)].contiguous()
    start = torch.zeros(len(groups), dtype=torch.int32, device="cuda")
    yahkv.kv8_append(dp, table2, start, vt, vt)                                              # chunk kernel
    got = dp.numpy()
    for s, grp in enumerate(groups):
        dw = got["vq"][:, s * 16].reshape(1024, 4)
        st = got["vs"][:, s * 16].view(np.uint16).reshape(1024, 2)
        for slot, j in enumerate(grp):
            assert np.array_equal(dw[64 * slot:64 * slot + 64], gold["v_dw"][j]), f"V tile {j}: codes (chunk kernel)"
            assert np.array_equal(st[64 * slot:64 * slot + 64], gold["v_st"][j]), f"V tile {j}: stats"
    dp2 = yahkv.Kv8Pools(g)
    for key in range(16):                                                                     # token by token
        yahkv.kv8_append(dp2, table2, start + key, vt[:, key:key + 1].contiguous(), vt[:, key:key + 1].contiguous())
    got2 = dp2.numpy()
    mine = [16 * s for s in range(len(groups))]
    assert np.array_equal(got2["vq"][:, mine], got["vq"][:, mine]) and np.array_equal(got2["vs"][:, mine], got["vs"][:, mine])


def test_kmean_bit_exact(yahkv, torch_gpu):
    torch = torch_gpu
    rng = np.random.default_rng(12)
    g = yahkv.kv8_geometry(12, 2, 6)
    dp = yahkv.Kv8Pools(g)
    k = (rng.standard_normal((3, 333, 2, 256)) * 3 + rng.standard_normal((2, 256))).astype(np.float32)
    table = torch.tensor([[4, 0], [2, 1], [5, 3]], dtype=torch.int32, device="cuda")
    n_valid = np.array([333, 100, 0], np.int32)
    for dtype in (torch.float32, torch.bfloat16):
        kt = torch.from_numpy(k).cuda().to(dtype)
        yahkv.kv8_kmean(dp, table, kt, torch.from_numpy(n_valid).cuda())
        km = dp.numpy()["km"]
        kh = kt.float().cpu().numpy()
        for s, page in enumerate((4, 2, 5)):
            n = min(333, max(int(n_valid[s]), 1))
            assert np.array_equal(km[page], kv8.kmean(kh[s, :n].reshape(n, 512))), f"sequence {s} ({dtype})"


def attend(yahkv, torch, dp, table, lens, q, gate=None, **kw):
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    out = yahkv.kv8_decode_attend(dp, table, sl, int(max(lens)), torch.from_numpy(q).cuda(), 1.0 / 16.0,
                                  None if gate is None else torch.from_numpy(gate).cuda(), **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def test_recipe_attention_against_the_checkers_own_result(yahkv, torch_gpu, rc):
    """part_q + reduce at pos 700 with a scrambled table and stale open-tile keys poisoned with 7.0 (:177), against the
    float64 result the checker itself compares with (:193-208)."""
    torch, g = torch_gpu, rc.g
    dp, table = dev_pools(yahkv, torch, rc, rc.n)
    arrs = dp.numpy()
    arrs["vo"][rc.ptab[rc.pos // 256]][:, rc.nk:] = np.float16(7.0).view(np.uint16)
    dp.load(arrs)
    out = attend(yahkv, torch, dp, table, [rc.n], rc.q[None], rc.gate[None])[0]
    err = rel_err(out, g["rc_ref"])
    print(f"kv8a16 decode vs the checker's dequantized model: {err:.2e} (the reference's own bar: 1e-4); "
          f"vs f16 KV {rel_err(out, g['rc_exact']):.2e}")
    assert err < TOL
    out2 = attend(yahkv, torch, dp, table, [rc.n], rc.q[None], None)[0]
    hp = host_pools(rc, rc.n)
    Kd, Vd = kv8.dense(hp, rc.ptab, rc.n)
    assert rel_err(out2, closed_form(Kd, Vd, rc.q, 1.0 / 16.0)) < TOL


@pytest.mark.parametrize("n", [1, 15, 16, 17, 64, 65, 255, 256, 257, 300, 1023, 1024])
def test_attention_at_tile_and_page_boundaries(yahkv, torch_gpu, rc, n):
    torch = torch_gpu
    dp, table = dev_pools(yahkv, torch, rc, n)
    hp = host_pools(rc, n)
    Kd, Vd = kv8.dense(hp, rc.ptab, n)
    out = attend(yahkv, torch, dp, table, [n], rc.q[None])[0]
    assert rel_err(out, closed_form(Kd, Vd, rc.q, 1.0 / 16.0)) < TOL
    if n == 1:                                             # one key: the output is that key's V row, to f16's last bit
        assert np.abs(out - np.repeat(Vd[0], 6, 0)).max() < 1e-6


def test_decode_steps_across_tiles_and_a_page(yahkv, torch_gpu, rc):
    """Steps 240 .. 275 after a chunk of 240: every step's output, and the pools at the end, against a token-by-token
    oracle. Crosses tile boundaries (a tile closes on 255, 271) and the page boundary at 256."""
    torch = torch_gpu
    n0, n1 = 240, 276
    dp, table = dev_pools(yahkv, torch, rc, n0, fill=0x11)
    hp = host_pools(rc, n0, fill=0x11)
    worst = 0.0
    for pos in range(n0, n1):
        kn = torch.from_numpy(rc.K[pos].astype(np.float32).reshape(1, 4, 256)).cuda()
        vn = torch.from_numpy(rc.V[pos].astype(np.float32).reshape(1, 4, 256)).cuda()
        sl = torch.tensor([pos + 1], dtype=torch.int32, device="cuda")
        out = yahkv.kv8_decode_step(dp, table, sl, pos + 1, kn, vn, torch.from_numpy(rc.q[None]).cuda(), 1.0 / 16.0)
        kv8.append(hp, rc.ptab[None], [pos], None, rc.K[None, pos:pos + 1].astype(np.float32), rc.V[None, pos:pos + 1].astype(np.float32))
        Kd, Vd = kv8.dense(hp, rc.ptab, pos + 1)
        worst = max(worst, rel_err(out.cpu().numpy()[0], closed_form(Kd, Vd, rc.q, 1.0 / 16.0)))
    assert worst < TOL, worst
    assert_pools_equal(dp, hp, "after 36 steps")
    # the step and the two separate calls agree
    dp2, _ = dev_pools(yahkv, torch, rc, n0, fill=0x11)
    for pos in range(n0, n0 + 20):
        kn = torch.from_numpy(rc.K[pos].reshape(1, 1, 4, 256)).cuda()
        vn = torch.from_numpy(rc.V[pos].reshape(1, 1, 4, 256)).cuda()
        yahkv.kv8_append(dp2, table, torch.tensor([pos], dtype=torch.int32, device="cuda"), kn, vn)
    hp2 = host_pools(rc, n0, fill=0x11)
    for pos in range(n0, n0 + 20):
        kv8.append(hp2, rc.ptab[None], [pos], None, rc.K[None, pos:pos + 1].astype(np.float32), rc.V[None, pos:pos + 1].astype(np.float32))
    assert_pools_equal(dp2, hp2, "20 one-token appends")


def test_ragged_batch_shared_pool(yahkv, torch_gpu):
    """Several sequences of ragged lengths in one shuffled pool: chunk appends with padded chunks (n_valid), a chunk that
    continues mid-tile, then attention with a gate; every row against the closed form, the pools against the oracle."""
    torch = torch_gpu
    rng = np.random.default_rng(21)
    lens = [5, 700, 16, 1300, 257, 2047, 1, 96]
    n_q, H = 12, 2
    pages = [(n + 40 + 255) // 256 for n in lens]
    P = sum(pages) + 3
    perm = rng.permutation(P).astype(np.int32)
    stride = max(pages)
    table = np.zeros((len(lens), stride), np.int32)
    o = 0
    for s, np_ in enumerate(pages):
        table[s, :np_] = perm[o:o + np_]
        o += np_
    g = yahkv.kv8_geometry(n_q, H, P)
    dp, hp = yahkv.Kv8Pools(g, 0x77), kv8.HostPools(kv8.geometry(n_q, H, P), 0x77)
    cap = max(lens)
    K = (rng.standard_normal((len(lens), cap, H, 256)) + 0.5 * rng.standard_normal((len(lens), 1, H, 256))).astype(np.float16)
    V = rng.standard_normal((len(lens), cap, H, 256)).astype(np.float16)
    t_table = torch.from_numpy(table).cuda()
    nv = np.array(lens, np.int32)
    Kt, Vt = torch.from_numpy(K).cuda(), torch.from_numpy(V).cuda()
    yahkv.kv8_kmean(dp, t_table, Kt, torch.from_numpy(nv).cuda())
    for s in range(len(lens)):
        hp.km[table[s, 0]] = kv8.kmean(K[s, :lens[s]].astype(np.float32).reshape(lens[s], H * 256))
    first = np.minimum(nv, 37).astype(np.int32)             # a first chunk that ends inside a tile, then the rest
    zero = torch.zeros(len(lens), dtype=torch.int32, device="cuda")
    yahkv.kv8_append(dp, t_table, zero, Kt[:, :37].contiguous(), Vt[:, :37].contiguous(), torch.from_numpy(first).cuda())
    kv8.append(hp, table, np.zeros(len(lens), np.int32), first, K[:, :37].astype(np.float32).reshape(len(lens), 37, -1),
               V[:, :37].astype(np.float32).reshape(len(lens), 37, -1))
    rest = (nv - first).astype(np.int32)
    yahkv.kv8_append(dp, t_table, torch.from_numpy(first).cuda(), Kt[:, 37:].contiguous(), Vt[:, 37:].contiguous(),
                     torch.from_numpy(rest).cuda())
    kv8.append(hp, table, first, rest, K[:, 37:].astype(np.float32).reshape(len(lens), cap - 37, -1),
               V[:, 37:].astype(np.float32).reshape(len(lens), cap - 37, -1))
    torch.cuda.synchronize()
    assert_pools_equal(dp, hp, "ragged chunks")
    q = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
    gate = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
    runs = []
    for kw in ({}, {}, {"opt": yahkv.DecodeOptions(deterministic=-1)}):    # the default twice, then tiles first come, first served
        out = attend(yahkv, torch, dp, t_table, lens, q, gate, **kw)
        runs.append(out)
        for s, n in enumerate(lens):
            Kd, Vd = kv8.dense(hp, table[s], n)
            assert rel_err(out[s], closed_form(Kd, Vd, q[s], 1.0 / 16.0, gate[s])) < TOL, (s, n)
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32))   # the default repeats bit for bit
    # a step for every sequence at once
    kn = rng.standard_normal((len(lens), H, 256)).astype(np.float32)
    vn = rng.standard_normal((len(lens), H, 256)).astype(np.float32)
    sl = torch.from_numpy(nv + 1).cuda()
    out = yahkv.kv8_decode_step(dp, t_table, sl, int(max(lens)) + 1, torch.from_numpy(kn).cuda(), torch.from_numpy(vn).cuda(),
                                torch.from_numpy(q).cuda().to(torch.bfloat16), 1.0 / 16.0).cpu().numpy()
    kv8.append(hp, table, nv, None, kn.reshape(len(lens), 1, -1), vn.reshape(len(lens), 1, -1))
    assert_pools_equal(dp, hp, "batched step")
    qb = torch.from_numpy(q).to(torch.bfloat16).float().numpy()
    for s, n in enumerate(lens):
        Kd, Vd = kv8.dense(hp, table[s], n + 1)
        assert rel_err(out[s], closed_form(Kd, Vd, qb[s], 1.0 / 16.0)) < TOL, (s, n)


def test_chunked_prefill_over_a_paged_prefix(yahkv, torch_gpu):
    """Two sequences with prefixes of different lengths (one ending inside a tile), a chunk appended to each, then the
    chunk's causal attention: against the closed form over the prefill-side decode (one f16 fma per element, every V
    tile from codes; gen_attn_fa.py:4648-4861)."""
    torch = torch_gpu
    rng = np.random.default_rng(31)
    n_q, H, chunk = 12, 2, 200
    prefix = [300, 77]
    pages = [(p + chunk + 255) // 256 for p in prefix]
    P = sum(pages) + 2
    perm = rng.permutation(P).astype(np.int32)
    table = np.zeros((2, max(pages)), np.int32)
    table[0, :pages[0]], table[1, :pages[1]] = perm[:pages[0]], perm[pages[0]:pages[0] + pages[1]]
    g = yahkv.kv8_geometry(n_q, H, P)
    dp, hp = yahkv.Kv8Pools(g, 0x21), kv8.HostPools(kv8.geometry(n_q, H, P), 0x21)
    cap = max(prefix)
    K = (rng.standard_normal((2, cap + chunk, H, 256)) + 0.7 * rng.standard_normal((2, 1, H, 256))).astype(np.float16)
    V = rng.standard_normal((2, cap + chunk, H, 256)).astype(np.float16)
    t_table = torch.from_numpy(table).cuda()
    pl = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    Kp, Vp = torch.from_numpy(K[:, :cap].copy()).cuda(), torch.from_numpy(V[:, :cap].copy()).cuda()
    yahkv.kv8_kmean(dp, t_table, Kp, pl)
    yahkv.kv8_append(dp, t_table, torch.zeros(2, dtype=torch.int32, device="cuda"), Kp, Vp, pl)
    Kc = np.stack([K[s, prefix[s]:prefix[s] + chunk] for s in range(2)])
    Vc = np.stack([V[s, prefix[s]:prefix[s] + chunk] for s in range(2)])
    yahkv.kv8_append(dp, t_table, pl, torch.from_numpy(Kc).cuda(), torch.from_numpy(Vc).cuda())
    for s in range(2):
        hp.km[table[s, 0]] = kv8.kmean(K[s, :prefix[s]].astype(np.float32).reshape(prefix[s], -1))
    kv8.append(hp, table, [0, 0], prefix, K[:, :cap].astype(np.float32).reshape(2, cap, -1), V[:, :cap].astype(np.float32).reshape(2, cap, -1))
    kv8.append(hp, table, prefix, None, Kc.astype(np.float32).reshape(2, chunk, -1), Vc.astype(np.float32).reshape(2, chunk, -1))
    torch.cuda.synchronize()
    assert_pools_equal(dp, hp, "prefix + chunk")
    q = torch.from_numpy(rng.standard_normal((2, chunk, n_q, 256)).astype(np.float32)).cuda().to(torch.bfloat16)
    gate = rng.standard_normal((2, chunk, n_q, 256)).astype(np.float32)
    out = yahkv.kv8_prefill_attend(dp, t_table, pl, max(prefix), q, 1.0 / 16.0, torch.from_numpy(gate).cuda(),
                                   out=torch.empty(q.shape, dtype=torch.float32, device="cuda")).cpu().numpy()
    qf = q.float().cpu().numpy()
    worst = 0.0
    for s in range(2):
        n = prefix[s] + chunk
        Kh, Vh = kv8.dense(hp, table[s], n, as_f16=True)
        for t in (0, 1, 15, 16, 63, 64, 128, chunk - 1):
            vis = prefix[s] + t + 1
            worst = max(worst, rel_err(out[s, t], closed_form(Kh[:vis], Vh[:vis], qf[s, t], 1.0 / 16.0, gate[s, t])))
    print(f"kv8a16 prefill vs the closed form over its own f16 decode: {worst:.2e}")
    assert worst < TOL


@pytest.mark.parametrize("bits", [8, 4])
def test_chunks_that_start_inside_a_tile_and_end_in_its_page(yahkv, torch_gpu, bits):
    """The chunk's first tile takes its earlier keys from the page's open tile, and the chunk's newest tile is written
    there: with first and newest tile in one page these are the same bytes, read and written inside one launch. Many
    sequences with such chunks (and some that start on a tile, end on one, or cross into the next page), three chunks
    one after the other, every buffer against the oracle after each."""
    torch = torch_gpu
    rng = np.random.default_rng(77)
    n_q, H, S = 8, 4, 96
    g = yahkv.kv8_geometry(n_q, H, 2 * S, bits, bits)
    dp, hp = yahkv.Kv8Pools(g, 0x33), kv8.HostPools(kv8.geometry(n_q, H, 2 * S, bits, bits), 0x33)
    table = rng.permutation(2 * S).astype(np.int32).reshape(S, 2)
    t_table = torch.from_numpy(table).cuda()
    pos = rng.integers(0, 40, S).astype(np.int32)
    pos[:4] = (0, 16, 5, 250)
    first = np.maximum(pos, 1)
    K0 = rng.standard_normal((S, 256, H, 256)).astype(np.float16)
    V0 = rng.standard_normal((S, 256, H, 256)).astype(np.float16)
    nv = torch.from_numpy(first).cuda()
    yahkv.kv8_kmean(dp, t_table, torch.from_numpy(K0).cuda(), nv)
    for s in range(S):
        hp.km[table[s, 0]] = kv8.kmean(K0[s, :first[s]].astype(np.float32).reshape(first[s], -1))
    # the keys before the first chunk, so that there is an open tile to read
    yahkv.kv8_append(dp, t_table, torch.zeros(S, dtype=torch.int32, device="cuda"), torch.from_numpy(K0).cuda(),
                     torch.from_numpy(V0).cuda(), torch.from_numpy(pos).cuda())
    kv8.append(hp, table, [0] * S, pos.tolist(), K0.astype(np.float32).reshape(S, 256, -1), V0.astype(np.float32).reshape(S, 256, -1))
    for step, chunk in enumerate((37, 64, 50)):
        n = rng.integers(2, chunk + 1, S).astype(np.int32)
        n[:3] = chunk
        K = rng.standard_normal((S, chunk, H, 256)).astype(np.float16)
        V = rng.standard_normal((S, chunk, H, 256)).astype(np.float16)
        yahkv.kv8_append(dp, t_table, torch.from_numpy(pos).cuda(), torch.from_numpy(K).cuda(), torch.from_numpy(V).cuda(),
                         torch.from_numpy(n).cuda())
        kv8.append(hp, table, pos.tolist(), n.tolist(), K.astype(np.float32).reshape(S, chunk, -1), V.astype(np.float32).reshape(S, chunk, -1))
        torch.cuda.synchronize()
        assert_pools_equal(dp, hp, f"chunk {step} of {chunk} rows")
        pos = pos + n


@pytest.mark.parametrize("seed,bits", [(1, 8), (2, 8), (3, 4), (4, 4)])
def test_random_appends_against_the_oracle(yahkv, torch_gpu, seed, bits):
    """Sequences that grow by calls of random length (one token, a few, several tiles, across pages), some rows of a
    call padding, f16 or bf16 or f32 rows: after every call all six buffers are the oracle's, byte for byte."""
    torch = torch_gpu
    rng = np.random.default_rng(1000 + seed)
    n_q, H = 8, 2
    S = int(rng.integers(3, 40))
    pages_each = 4
    g = yahkv.kv8_geometry(n_q, H, S * pages_each + 1, bits, bits)
    dp, hp = yahkv.Kv8Pools(g, 0x17), kv8.HostPools(kv8.geometry(n_q, H, S * pages_each + 1, bits, bits), 0x17)
    table = rng.permutation(S * pages_each + 1)[:S * pages_each].astype(np.int32).reshape(S, pages_each)
    t_table = torch.from_numpy(table).cuda()
    pos = np.zeros(S, np.int32)
    cap = pages_each * 256
    first = True
    for call in range(9):
        n_new = int(rng.choice([1, 1, 2, 5, 16, 33, 100, 257, 300]))
        n = rng.integers(0 if not first else 1, n_new + 1, S).astype(np.int32)
        n = np.minimum(n, cap - pos).astype(np.int32)
        n[0] = min(n_new, cap - pos[0])
        dt = [np.float16, "bf16", np.float32][call % 3]
        K = (rng.standard_normal((S, n_new, H, 256)) + 0.3).astype(np.float32)
        V = rng.standard_normal((S, n_new, H, 256)).astype(np.float32)
        if dt == "bf16":
            tk, tv = torch.from_numpy(K).cuda().to(torch.bfloat16), torch.from_numpy(V).cuda().to(torch.bfloat16)
            K, V = tk.float().cpu().numpy(), tv.float().cpu().numpy()
        else:
            K, V = K.astype(dt), V.astype(dt)
            tk, tv = torch.from_numpy(K).cuda(), torch.from_numpy(V).cuda()
        if first:                                      # the channel means from each sequence's first rows
            yahkv.kv8_kmean(dp, t_table, tk, torch.from_numpy(n).cuda())
            for s in range(S):
                hp.km[table[s, 0]] = kv8.kmean(K[s, :max(n[s], 1)].astype(np.float32).reshape(max(n[s], 1), -1))
            first = False
        yahkv.kv8_append(dp, t_table, torch.from_numpy(pos).cuda(), tk, tv, torch.from_numpy(n).cuda())
        kv8.append(hp, table, pos.tolist(), n.tolist(), K.astype(np.float32).reshape(S, n_new, -1), V.astype(np.float32).reshape(S, n_new, -1))
        torch.cuda.synchronize()
        assert_pools_equal(dp, hp, f"seed {seed}, call {call}: {n_new} rows of {dt}")
        pos = pos + n


def test_refusals(yahkv, torch_gpu):
    torch = torch_gpu
    g = yahkv.kv8_geometry(24, 4, 2)
    dp = yahkv.Kv8Pools(g)
    table = torch.zeros((1, 2), dtype=torch.int32, device="cuda")
    k = torch.zeros((1, 1, 4, 256), device="cuda")
    st = dp.struct()
    st.vopen_bytes -= 1                                    # a pool shorter than the geometry needs
    import ctypes as C
    rc_ = yahkv.lib.yahkv_kv8_append(C.byref(g), C.byref(st), table.data_ptr(), 2, table.data_ptr(), None, 1, 1,
                                     k.data_ptr(), k.data_ptr(), 0, None)
    assert rc_ == -1
    bad = yahkv.Geometry(yahkv.KV8A16, 24, 4, 128, 256, 2)
    assert yahkv.lib.yahkv_kv8_kq_bytes(C.byref(bad)) == 0
    q8 = yahkv.geometry(yahkv.Q8_0, 24, 4, 256, 64, 2)
    assert yahkv.lib.yahkv_kv8_kq_bytes(C.byref(q8)) == 0   # the quantized block formats have their own functions
    with pytest.raises(yahkv.YahkvError):
        yahkv.kv8_decode_attend(dp, table, torch.ones(1, dtype=torch.int32, device="cuda"), 1,
                                torch.zeros((1, 24, 256), device="cuda"), 0.0625, opt=yahkv.DecodeOptions(one_launch=1))


def test_xcd_calibration_for_these_formats(yahkv, torch_gpu):
    """yahkv_kv8_decode_calibrate returns shares of the XCDs' speeds that leave the results where they were."""
    torch = torch_gpu
    rng = np.random.default_rng(41)
    lens = [int(x) for x in rng.integers(3000, 20000, 24)]
    n_q, H = 24, 4
    pages = [(n + 255) // 256 for n in lens]
    P = sum(pages)
    table = np.zeros((len(lens), max(pages)), np.int32)
    perm, o = rng.permutation(P).astype(np.int32), 0
    for s, np_ in enumerate(pages):
        table[s, :np_] = perm[o:o + np_]
        o += np_
    g = yahkv.kv8_geometry(n_q, H, P)
    dp = yahkv.Kv8Pools(g)
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(3)
    for s, n in enumerate(lens):
        k = torch.randn((1, n, H, 256), generator=gen, device="cuda").to(torch.bfloat16)
        v = torch.randn((1, n, H, 256), generator=gen, device="cuda").to(torch.bfloat16)
        yahkv.kv8_kmean(dp, t_table[s:s + 1], k)
        yahkv.kv8_append(dp, t_table[s:s + 1], torch.zeros(1, dtype=torch.int32, device="cuda"), k, v)
    q = torch.randn((len(lens), n_q, 256), generator=gen, device="cuda")
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    before = yahkv.kv8_decode_attend(dp, t_table, sl, max(lens), q, 0.0625).cpu().numpy()
    opt = yahkv.decode_options()
    ws = torch.empty(yahkv.lib.yahkv_kv8_decode_workspace_bytes(g, len(lens), max(lens), opt), dtype=torch.uint8, device="cuda")
    w = yahkv.kv8_decode_calibrate(dp, t_table, sl, max(lens), q, ws, opt, rounds=2)
    assert len(w) == 8 and max(w) == 10000 and min(w) >= 5000, w
    after = yahkv.kv8_decode_attend(dp, t_table, sl, max(lens), q, 0.0625, workspace=ws, opt=opt).cpu().numpy()
    assert rel_err(after, before) < 5e-4


@pytest.mark.parametrize("n_q,H,kb", [(4, 1, 8), (6, 3, 8), (16, 8, 8), (16, 8, 4), (6, 3, 4)])
def test_other_kv_head_counts(yahkv, torch_gpu, n_q, H, kb):
    """The split-K kernel deals the kv heads of a tile to a workgroup's eight waves where the head count divides 8 (one,
    two, four, eight heads) and cuts the work by (sequence, kv head) otherwise (three): both against the oracle, on ragged
    lengths with a step."""
    torch = torch_gpu
    rng = np.random.default_rng(50 + H + kb)
    lens = [300, 1, 2100, 17, 700]
    pages = [(n + 1 + 255) // 256 for n in lens]
    P = sum(pages) + 1
    perm, o = rng.permutation(P).astype(np.int32), 0
    table = np.zeros((len(lens), max(pages)), np.int32)
    for s, np_ in enumerate(pages):
        table[s, :np_] = perm[o:o + np_]
        o += np_
    g = yahkv.kv8_geometry(n_q, H, P, kb, kb)
    dp, hp = yahkv.Kv8Pools(g, 0x42), kv8.HostPools(kv8.geometry(n_q, H, P, kb, kb), 0x42)
    cap = max(lens)
    K = (rng.standard_normal((len(lens), cap, H, 256)) + 0.4).astype(np.float16)
    V = rng.standard_normal((len(lens), cap, H, 256)).astype(np.float16)
    t_table = torch.from_numpy(table).cuda()
    nv = np.array(lens, np.int32)
    yahkv.kv8_kmean(dp, t_table, torch.from_numpy(K).cuda(), torch.from_numpy(nv).cuda())
    for s in range(len(lens)):
        hp.km[table[s, 0]] = kv8.kmean(K[s, :lens[s]].astype(np.float32).reshape(lens[s], H * 256))
    yahkv.kv8_append(dp, t_table, torch.zeros(len(lens), dtype=torch.int32, device="cuda"), torch.from_numpy(K).cuda(),
                     torch.from_numpy(V).cuda(), torch.from_numpy(nv).cuda())
    kv8.append(hp, table, np.zeros(len(lens), np.int32), nv, K.astype(np.float32).reshape(len(lens), cap, -1),
               V.astype(np.float32).reshape(len(lens), cap, -1))
    assert_pools_equal(dp, hp, f"{H} kv heads")
    q = rng.standard_normal((len(lens), n_q, 256)).astype(np.float32)
    out = attend(yahkv, torch, dp, t_table, lens, q)
    rot = (lambda x: kv8.rotate_q(x)) if kb == 4 else (lambda x: x)
    for s, n in enumerate(lens):
        Kd, Vd = kv8.dense(hp, table[s], n)
        assert rel_err(out[s], closed_form(Kd, Vd, rot(q[s]), 1.0 / 16.0)) < TOL, (s, n)
    kn = rng.standard_normal((len(lens), H, 256)).astype(np.float32)
    vn = rng.standard_normal((len(lens), H, 256)).astype(np.float32)
    out = yahkv.kv8_decode_step(dp, t_table, torch.from_numpy(nv + 1).cuda(), cap + 1, torch.from_numpy(kn).cuda(),
                                torch.from_numpy(vn).cuda(), torch.from_numpy(q).cuda(), 1.0 / 16.0).cpu().numpy()
    kv8.append(hp, table, nv, None, kn.reshape(len(lens), 1, -1), vn.reshape(len(lens), 1, -1))
    assert_pools_equal(dp, hp, "step")
    for s, n in enumerate(lens):
        Kd, Vd = kv8.dense(hp, table[s], n + 1)
        assert rel_err(out[s], closed_form(Kd, Vd, rot(q[s]), 1.0 / 16.0)) < TOL, (s, n)


@pytest.mark.parametrize("kb,vb", [(8, 8), (4, 4)])
def test_page_copies_and_slots(yahkv, torch_gpu, rc, kb, vb):
    """yahkv_kv8_copy_pages moves a page's share of all six buffers; a slot's body is the sequence's pools with the identity
    page table (the oracle's pools_of_sequence, buffer after buffer); it unpacks into other pages of another pool, where
    the attention gives the same bits; headers of another geometry are refused."""
    torch = torch_gpu
    n = 700
    g = yahkv.kv8_geometry(24, 4, rc.T // 256, kb, vb)
    dp = yahkv.Kv8Pools(g, 0x5A)
    arrs = dp.numpy()
    arrs["km"][rc.ptab[0]] = rc.m
    dp.load(arrs)
    table = torch.from_numpy(rc.ptab[None].copy()).cuda()
    yahkv.kv8_append(dp, table, torch.zeros(1, dtype=torch.int32, device="cuda"),
                     torch.from_numpy(rc.K[None, :n].reshape(1, n, 4, 256)).cuda(), torch.from_numpy(rc.V[None, :n].reshape(1, n, 4, 256)).cuda())
    q = torch.from_numpy(rc.q[None]).cuda()
    sl = torch.tensor([n], dtype=torch.int32, device="cuda")
    want = yahkv.kv8_decode_attend(dp, table, sl, n, q, 0.0625).cpu().numpy()
    # the slot: header, then pools of three pages with the identity table
    slot = yahkv.kv8_slot_pack(dp, table[0], 3, n)
    host = slot.cpu().numpy()
    assert yahkv.kv8_slot_check(g, host) == (3, n)
    hp, _ = kv8.pools_of_sequence(dp, rc.ptab, n)
    body = b"".join(np.ascontiguousarray(getattr(hp, name)).tobytes() for name in ("kq", "ks", "km", "vq", "vs", "vo"))
    assert host[64:].tobytes() == body
    other = yahkv.kv8_geometry(16, 2, rc.T // 256, kb, vb)
    with pytest.raises(yahkv.YahkvError):
        yahkv.kv8_slot_check(other, host)
    with pytest.raises(yahkv.YahkvError):
        yahkv.kv8_slot_check(g, host[:-16])
    # into pages (6, 1, 4) of a pool of seven pages
    g7 = yahkv.kv8_geometry(24, 4, 7, kb, vb)
    dp7 = yahkv.Kv8Pools(g7, 0x33)
    row = torch.tensor([6, 1, 4], dtype=torch.int32, device="cuda")
    yahkv.kv8_slot_unpack(dp7, row, 3, slot)
    got = yahkv.kv8_decode_attend(dp7, row[None], sl, n, q, 0.0625).cpu().numpy()
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    a7 = dp7.numpy()
    for untouched in (0, 2, 3, 5):
        assert np.all(a7["kq"][untouched * 256:untouched * 256 + 256] == 0x33333333)
        assert np.all(a7["vq"][:, untouched * 16:untouched * 16 + 16] == 0x33333333) and np.all(a7["vo"][untouched] == 0x3333)
    # a page copied inside the pools carries all six buffers' shares
    yahkv.kv8_copy_pages(dp7, torch.tensor([4], dtype=torch.int32, device="cuda"), torch.tensor([0], dtype=torch.int32, device="cuda"))
    b7 = dp7.numpy()
    for name in ("kq", "ks"):
        assert np.array_equal(b7[name][0:256], a7[name][4 * 256:5 * 256]), name
    assert np.array_equal(b7["vq"][:, 0:16], a7["vq"][:, 64:80]) and np.array_equal(b7["vs"][:, 0:16], a7["vs"][:, 64:80])
    assert np.array_equal(b7["vo"][0], a7["vo"][4]) and np.array_equal(b7["km"][0].view(np.uint32), a7["km"][4].view(np.uint32))
    got2 = yahkv.kv8_decode_attend(dp7, torch.tensor([[6, 1, 0]], dtype=torch.int32, device="cuda"), sl, n, q, 0.0625).cpu().numpy()
    assert np.array_equal(got2.view(np.uint32), want.view(np.uint32))
