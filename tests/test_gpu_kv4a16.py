"""kv4a16 (and the mixes k8v4 / k4v8), the reference's 4-bit KV format, on the GPU through the C ABI (yahkv_kv8_* with
a 4-bit geometry): pools bit for bit against the CPU oracle restating the reference's kernels, the V side and the
"exact" K rows also bit for bit against the fixtures written from the reference's numpy model
(tests/golden/kv4a16_vectors.npz, dattn_q_check.py:52-256); attention against the float64 closed form over the
dequantized model with the rotated query, held to 2e-3."""
import numpy as np
import pytest

import kv8_recipe
from helpers import closed_form, rel_err
from oracle import kv8

pytestmark = pytest.mark.gpu
TOL = 2e-3
FORMATS = [(4, 4), (8, 4), (4, 8)]


@pytest.fixture(scope="module")
def rc():
    return kv8_recipe.load(4)


def dev_pools(yahkv, torch, rc, n_tokens, fill=0, kb=4, vb=4):
    g = yahkv.kv8_geometry(24, 4, rc.T // 256, kb, vb)
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


def host_pools(rc, n_tokens, fill=0, kb=4, vb=4):
    hp = kv8.HostPools(kv8.geometry(24, 4, rc.T // 256, kb, vb), fill)
    hp.km[rc.ptab[0]] = rc.m
    if n_tokens:
        kv8.append(hp, rc.ptab[None], [0], None, rc.K[None, :n_tokens].astype(np.float32), rc.V[None, :n_tokens].astype(np.float32))
    return hp


def assert_pools_equal(dp, hp, what=""):
    got = dp.numpy()
    for name, want in hp.arrays().items():
        if name == "km":
            assert np.array_equal(got[name].view(np.uint32), want.view(np.uint32)), f"{what}: km"
        else:
            assert got[name].shape == want.shape, f"{what}: {name} shape {got[name].shape} against {want.shape}"
            bad = np.argwhere(got[name] != want)
            assert bad.size == 0, (f"{what}: {name} differs from the oracle at {bad[:4].tolist()} ({len(bad)} places): got "
                                   f"{[hex(int(got[name][tuple(b)])) for b in bad[:4]]} want {[hex(int(want[tuple(b)])) for b in bad[:4]]}")


@pytest.mark.parametrize("kb,vb", FORMATS)
def test_recipe_chunk_append_bit_exact(yahkv, torch_gpu, rc, kb, vb):
    """The checker's pools from one chunk append against the oracle (every byte, the poison fill included); with 4-bit V
    also against the fixture's stats, code digest and open tile."""
    g = rc.g
    dp, _ = dev_pools(yahkv, torch_gpu, rc, rc.n, fill=0x5A, kb=kb, vb=vb)
    torch_gpu.cuda.synchronize()
    assert_pools_equal(dp, host_pools(rc, rc.n, fill=0x5A, kb=kb, vb=vb), f"chunk of 701, k{kb}v{vb}")
    got = dp.numpy()
    if vb == 4:
        closed = [kv8_recipe.ptile(rc, t) for t in range(rc.curt)]
        vq = np.zeros_like(got["vq"])
        vq[:, closed] = got["vq"][:, closed]
        assert np.array_equal(kv8_recipe.sha(vq), g["rc_vq_sha"])
        assert np.array_equal(got["vs"][:, closed].view(np.uint16).reshape(4, len(closed), 256, 2), g["rc_vs"][:, closed])
        assert np.array_equal(got["vo"][rc.ptab[rc.pos // 256]][:, :rc.nk], g["rc_vopen"][:, :rc.nk])


@pytest.mark.parametrize("kb,vb", FORMATS)
def test_recipe_kappend_and_vappend(yahkv, torch_gpu, rc, kb, vb):
    """dattn_q_check.py:210-250 with 4-bit codes: the K append at position 517; the V append mid-tile and on the tile's
    16th key (4-bit V: the closing tile's codes and stats bit for bit against the fixture)."""
    torch, g = torch_gpu, rc.g
    dp, table = dev_pools(yahkv, torch, rc, rc.n, fill=0x33, kb=kb, vb=vb)
    hp = host_pools(rc, rc.n, fill=0x33, kb=kb, vb=vb)
    p2 = int(g["rc_p2"])
    kx = torch.from_numpy(g["rc_kx"].reshape(1, 1, 4, 256)).cuda()
    yahkv.kv8_append(dp, table, torch.tensor([p2], dtype=torch.int32, device="cuda"), kx, torch.zeros_like(kx))
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
        if p3 % 16 == 15 and vb == 4:
            assert np.array_equal(got["vq"][:, pt], g["rc_v3_dw"]), "closing key: codes"
            assert np.array_equal(got["vs"][:, pt].view(np.uint16).reshape(4, 256, 2), g["rc_v3_st"]), "closing key: stats"
        kv8.append(hp, rc.ptab[None], [p3], None, rc.K[None, p3:p3 + 1].astype(np.float32), g[f"rc_vx_{case}"][None, None])
        assert_pools_equal(dp, hp, f"vappend at {p3}")


def test_directed_rows_and_tiles_through_the_kernels(yahkv, torch_gpu):
    """The fixture's exact K rows (ties, dead groups, negative lows: the rotation is exact in any order, so the reference's
    numpy model pins every bit), its random rows (against the oracle bit for bit, against the model within the rotation's
    rounding) and its V tiles, through the one-token and the chunk kernels."""
    torch = torch_gpu
    gold = kv8_recipe.golden(4)
    k_in = np.concatenate([gold["kx_in"], gold["kr_in"]])
    k_mean = np.concatenate([np.zeros_like(gold["kx_in"]), gold["kr_mean"]])
    nx, n = gold["kx_in"].shape[0], k_in.shape[0]
    g = yahkv.kv8_geometry(24, 4, n, 4, 4)                 # one sequence (one page) per row: each has its own means
    dp = yahkv.Kv8Pools(g)
    arrs = dp.numpy()
    arrs["km"][:] = k_mean
    dp.load(arrs)
    table = torch.arange(n, dtype=torch.int32, device="cuda").reshape(n, 1)
    k = torch.from_numpy(k_in.reshape(n, 1, 4, 256)).cuda()
    k2 = torch.cat([k, k], 1)                              # the chunk kernel: the same row twice, at positions 1 and 2
    yahkv.kv8_append(dp, table, torch.zeros(n, dtype=torch.int32, device="cuda"), k, torch.zeros_like(k))
    yahkv.kv8_append(dp, table, torch.ones(n, dtype=torch.int32, device="cuda"), k2, torch.zeros_like(k2))
    got = dp.numpy()
    for i in range(n):
        dw, sc = kv8.quant_k4(k_in[i], k_mean[i])
        for pos, kern in ((0, "one-token"), (1, "chunk"), (2, "chunk")):
            assert np.array_equal(got["kq"][i * 256 + pos], dw), f"K row {i}: codes ({kern} kernel) against the oracle"
            assert np.array_equal(got["ks"][i * 256 + pos].view(np.uint16), sc), f"K row {i}: scales ({kern} kernel)"
        if i < nx:
            assert np.array_equal(got["kq"][i * 256], gold["kx_dw"][i]), f"exact K row {i}: codes against the fixture"
            assert np.array_equal(got["ks"][i * 256].view(np.uint16), gold["kx_sc"][i]), f"exact K row {i}: scales"
    # V: sixteen 64-channel tiles side by side make one 1024-channel tile
    nt = gold["v_in"].shape[0]
    tiles = gold["v_in"].view(np.float16)
    reps = -(-nt // 16) * 16
    idx = np.arange(reps) % nt
    wide = tiles[idx].reshape(reps // 16, 16, 16, 64).transpose(0, 2, 1, 3).reshape(reps // 16, 16, 1024)   # [seq][key][1024]
    ns = wide.shape[0]
    g2 = yahkv.kv8_geometry(24, 4, ns, 4, 4)
    dp2 = yahkv.Kv8Pools(g2)
    table2 = torch.arange(ns, dtype=torch.int32, device="cuda").reshape(ns, 1)
    v = torch.from_numpy(wide.reshape(ns, 16, 4, 256).copy()).cuda()
    yahkv.kv8_append(dp2, table2, torch.zeros(ns, dtype=torch.int32, device="cuda"), torch.zeros_like(v), v)
    got2 = dp2.numpy()
    for s in range(ns):
        vq = got2["vq"][:, 16 * s].reshape(1024, 2)
        vs = got2["vs"][:, 16 * s].reshape(1024).view(np.uint16).reshape(1024, 2)
        for j in range(16):
            i = idx[16 * s + j]
            assert np.array_equal(vq[64 * j:64 * j + 64], gold["v_dw"][i]), f"V tile {i}: codes (chunk kernel)"
            assert np.array_equal(vs[64 * j:64 * j + 64], gold["v_st"][i]), f"V tile {i}: stats"
    # the same tiles key by key through the one-token kernel: the 16th key closes the tile
    dp3 = yahkv.Kv8Pools(g2)
    for key in range(16):
        yahkv.kv8_append(dp3, table2, torch.full((ns,), key, dtype=torch.int32, device="cuda"),
                         torch.zeros_like(v[:, :1]), v[:, key:key + 1].contiguous())
    got3 = dp3.numpy()
    assert np.array_equal(got3["vq"][:, ::16], got2["vq"][:, ::16]) and np.array_equal(got3["vs"][:, ::16], got2["vs"][:, ::16])


def attend(yahkv, torch, dp, table, lens, q, gate=None, **kw):
    sl = torch.tensor(lens, dtype=torch.int32, device="cuda")
    out = yahkv.kv8_decode_attend(dp, table, sl, int(max(lens)), torch.from_numpy(q).cuda(), 1.0 / 16.0,
                                  None if gate is None else torch.from_numpy(gate).cuda(), **kw)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def model_attention(hp, table_row, n, q, gate=None):
    """float64 closed form over the oracle's dequantized model; with 4-bit K against the rotated query rounded to f16, as
    the kernels hold it (the rounding is part of the computation the result is held to 2e-3 for, not of the model)."""
    Kd, Vd = kv8.dense(hp, table_row, n)
    qx = kv8.rotate_q(q) if hp.geom.k_bits == 4 else q
    return closed_form(Kd, Vd, qx, 1.0 / 16.0, gate)


def test_recipe_attention_against_the_checkers_own_result(yahkv, torch_gpu, rc):
    """part_q + reduce at pos 700 with a scrambled table and stale open-tile keys poisoned with 7.0, against the float64
    result the checker itself compares with (dattn_q_check.py:193-208, K4 against the rotated query)."""
    torch, g = torch_gpu, rc.g
    dp, table = dev_pools(yahkv, torch, rc, rc.n)
    arrs = dp.numpy()
    arrs["vo"][rc.ptab[rc.pos // 256]][:, rc.nk:] = np.float16(7.0).view(np.uint16)
    dp.load(arrs)
    out = attend(yahkv, torch, dp, table, [rc.n], rc.q[None], rc.gate[None])[0]
    err = rel_err(out, g["rc_ref"])
    print(f"kv4a16 decode vs the checker's dequantized model: {err:.2e}; vs f16 KV {rel_err(out, g['rc_exact']):.2e}")
    assert err < TOL
    out2 = attend(yahkv, torch, dp, table, [rc.n], rc.q[None], None)[0]
    assert rel_err(out2, model_attention(host_pools(rc, rc.n), rc.ptab, rc.n, rc.q)) < TOL


@pytest.mark.parametrize("kb,vb", FORMATS)
@pytest.mark.parametrize("n", [1, 15, 16, 17, 64, 65, 255, 256, 257, 300, 1023, 1024])
def test_attention_at_tile_and_page_boundaries(yahkv, torch_gpu, rc, n, kb, vb):
    torch = torch_gpu
    dp, table = dev_pools(yahkv, torch, rc, n, kb=kb, vb=vb)
    hp = host_pools(rc, n, kb=kb, vb=vb)
    out = attend(yahkv, torch, dp, table, [n], rc.q[None])[0]
    assert rel_err(out, model_attention(hp, rc.ptab, n, rc.q)) < TOL


@pytest.mark.parametrize("kb,vb", FORMATS)
def test_decode_steps_across_tiles_and_a_page(yahkv, torch_gpu, rc, kb, vb):
    """Steps 240 .. 275 after a chunk of 240: every step's output, and the pools at the end, against a token-by-token
    oracle. Crosses tile boundaries (a tile closes on 255, 271) and the page boundary at 256."""
    torch = torch_gpu
    n0, n1 = 240, 276
    dp, table = dev_pools(yahkv, torch, rc, n0, fill=0x11, kb=kb, vb=vb)
    hp = host_pools(rc, n0, fill=0x11, kb=kb, vb=vb)
    worst = 0.0
    for pos in range(n0, n1):
        kn = torch.from_numpy(rc.K[pos].astype(np.float32).reshape(1, 4, 256)).cuda()
        vn = torch.from_numpy(rc.V[pos].astype(np.float32).reshape(1, 4, 256)).cuda()
        sl = torch.tensor([pos + 1], dtype=torch.int32, device="cuda")
        out = yahkv.kv8_decode_step(dp, table, sl, pos + 1, kn, vn, torch.from_numpy(rc.q[None]).cuda(), 1.0 / 16.0)
        kv8.append(hp, rc.ptab[None], [pos], None, rc.K[None, pos:pos + 1].astype(np.float32), rc.V[None, pos:pos + 1].astype(np.float32))
        worst = max(worst, rel_err(out.cpu().numpy()[0], model_attention(hp, rc.ptab, pos + 1, rc.q)))
    assert worst < TOL, worst
    assert_pools_equal(dp, hp, "after 36 steps")


@pytest.mark.parametrize("kb,vb", FORMATS)
def test_ragged_batch_shared_pool(yahkv, torch_gpu, kb, vb):
    """Several sequences of ragged lengths in one shuffled pool: chunk appends with padded chunks (n_valid), a chunk that
    continues mid-tile, then attention with a gate; every row against the closed form, the pools against the oracle; the
    default repeats bit for bit; then a step for every sequence at once."""
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
    g = yahkv.kv8_geometry(n_q, H, P, kb, vb)
    dp, hp = yahkv.Kv8Pools(g, 0x77), kv8.HostPools(kv8.geometry(n_q, H, P, kb, vb), 0x77)
    cap = max(lens)
    K = (rng.standard_normal((len(lens), cap, H, 256)) + 0.5 * rng.standard_normal((len(lens), 1, H, 256))).astype(np.float16)
    V = rng.standard_normal((len(lens), cap, H, 256)).astype(np.float16)
    t_table = torch.from_numpy(table).cuda()
    nv = np.array(lens, np.int32)
    Kt, Vt = torch.from_numpy(K).cuda(), torch.from_numpy(V).cuda()
    yahkv.kv8_kmean(dp, t_table, Kt, torch.from_numpy(nv).cuda())
    for s in range(len(lens)):
        hp.km[table[s, 0]] = kv8.kmean(K[s, :lens[s]].astype(np.float32).reshape(lens[s], H * 256))
    first = np.minimum(nv, 37).astype(np.int32)
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
    for kw in ({}, {}, {"opt": yahkv.DecodeOptions(deterministic=-1)}):
        out = attend(yahkv, torch, dp, t_table, lens, q, gate, **kw)
        runs.append(out)
        for s, n in enumerate(lens):
            assert rel_err(out[s], model_attention(hp, table[s], n, q[s], gate[s])) < TOL, (s, n)
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32))
    kn = rng.standard_normal((len(lens), H, 256)).astype(np.float32)
    vn = rng.standard_normal((len(lens), H, 256)).astype(np.float32)
    sl = torch.from_numpy(nv + 1).cuda()
    out = yahkv.kv8_decode_step(dp, t_table, sl, int(max(lens)) + 1, torch.from_numpy(kn).cuda(), torch.from_numpy(vn).cuda(),
                                torch.from_numpy(q).cuda().to(torch.bfloat16), 1.0 / 16.0).cpu().numpy()
    kv8.append(hp, table, nv, None, kn.reshape(len(lens), 1, -1), vn.reshape(len(lens), 1, -1))
    assert_pools_equal(dp, hp, "batched step")
    qb = torch.from_numpy(q).to(torch.bfloat16).float().numpy()
    for s, n in enumerate(lens):
        assert rel_err(out[s], model_attention(hp, table[s], n + 1, qb[s])) < TOL, (s, n)


@pytest.mark.parametrize("kb,vb", FORMATS)
def test_chunked_prefill_over_a_paged_prefix(yahkv, torch_gpu, kb, vb):
    """Two sequences with prefixes of different lengths (one ending inside a tile), a chunk appended to each, then the
    chunk's causal attention: against the closed form over the prefill-side decode (one f16 fma per element, every V
    tile from codes; yah_kdeq4 / yah_vdeq4) with, for 4-bit K, the query rotated and rounded to f16 as yah_qrot leaves it."""
    torch = torch_gpu
    rng = np.random.default_rng(31)
    n_q, H, chunk = 12, 2, 200
    prefix = [300, 77]
    pages = [(p + chunk + 255) // 256 for p in prefix]
    P = sum(pages) + 2
    perm = rng.permutation(P).astype(np.int32)
    table = np.zeros((2, max(pages)), np.int32)
    table[0, :pages[0]], table[1, :pages[1]] = perm[:pages[0]], perm[pages[0]:pages[0] + pages[1]]
    g = yahkv.kv8_geometry(n_q, H, P, kb, vb)
    dp, hp = yahkv.Kv8Pools(g, 0x21), kv8.HostPools(kv8.geometry(n_q, H, P, kb, vb), 0x21)
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
    if kb == 4:
        qf = kv8.rotate_q(qf).astype(np.float16).astype(np.float32)
    worst = 0.0
    for s in range(2):
        n = prefix[s] + chunk
        Kh, Vh = kv8.dense(hp, table[s], n, as_f16=True)
        for t in (0, 1, 15, 16, 63, 64, 128, chunk - 1):
            vis = prefix[s] + t + 1
            worst = max(worst, rel_err(out[s, t], closed_form(Kh[:vis], Vh[:vis], qf[s, t], 1.0 / 16.0, gate[s, t])))
    print(f"k{kb}v{vb} prefill vs the closed form over its own f16 decode: {worst:.2e}")
    assert worst < TOL


def test_refusals(yahkv, torch_gpu):
    import ctypes as C
    bad = yahkv.Geometry(yahkv.KV4A16, 24, 4, 128, 256, 2)
    assert yahkv.lib.yahkv_kv8_kq_bytes(C.byref(bad)) == 0
    g = yahkv.kv8_geometry(24, 4, 2, 4, 4)
    assert yahkv.lib.yahkv_kv8_kq_bytes(C.byref(g)) == 2 * 256 * 512 and yahkv.lib.yahkv_kv8_ks_bytes(C.byref(g)) == 2 * 256 * 128
    assert yahkv.lib.yahkv_kv8_vq_bytes(C.byref(g)) == 4 * 32 * 256 * 8 and yahkv.lib.yahkv_kv8_vs_bytes(C.byref(g)) == 4 * 32 * 256 * 4
    dp = yahkv.Kv8Pools(yahkv.kv8_geometry(24, 4, 2, 8, 8))          # 8-bit pools are too short for... no: K is longer; V too
    g84 = yahkv.kv8_geometry(24, 4, 2, 4, 4)
    small = yahkv.Kv8Pools(g84)
    table = torch_gpu.zeros((1, 2), dtype=torch_gpu.int32, device="cuda")
    k = torch_gpu.zeros((1, 1, 4, 256), device="cuda")
    st = small.struct()
    g88 = yahkv.kv8_geometry(24, 4, 2, 8, 8)                         # 4-bit pools handed over with an 8-bit geometry
    rc_ = yahkv.lib.yahkv_kv8_append(C.byref(g88), C.byref(st), table.data_ptr(), 2, table.data_ptr(), None, 1, 1,
                                     k.data_ptr(), k.data_ptr(), 0, None)
    assert rc_ == -1
    del dp
