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
