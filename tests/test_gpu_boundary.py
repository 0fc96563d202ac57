"""The decode attention's boundary behaviour through the C ABI: the deterministic mode gives the same bits on every
call, queries beyond the f16 range saturate instead of poisoning the row, f32 queries are taken as the reference's
kernels take them, and the XCD calibration returns shares that leave the results unchanged."""
import numpy as np
import pytest

import oracle
from helpers import rel_err, to_bf16_f32
from test_gpu_decode import closed, gpu_attend, setup

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.mark.parametrize("fmt", [8, 4])
def test_decode_repeats_bit_for_bit(yahkv, torch_gpu, fmt):
    """The waves take a workgroup's tiles in a fixed pattern (the default, and what opt.deterministic > 0 asks for by
    name): the same bytes in give the same bits out, call after call, which makes a hash of the output a regression check
    as the reference's attn_bench uses its FNV hash (engine/run/attn_bench.cc:174-176; the reference treats bit-identity
    of a forward as a test, docs/build-and-run.md:259-260). Long sequences, so that every wave has several tiles."""
    torch = torch_gpu
    lens = [40000, 9000, 64, 20001, 1, 0, 5000, 12345]
    g, table, host, dev, rng = setup(yahkv, torch, fmt, 24, 4, 256, 64, lens, seed=fmt + 31)
    q = to_bf16_f32(rng.standard_normal((len(lens), 24, 256)))
    opt = yahkv.decode_options(deterministic=True)
    runs = [gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, opt=opt) for _ in range(3)]
    runs += [gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625) for _ in range(3)]       # no options: the same pattern
    for r in runs[1:]:
        assert np.array_equal(r.view(np.uint32), runs[0].view(np.uint32))
    assert rel_err(runs[0], oracle.decode_attend(host, table, lens, q, 0.0625)) < TOL
    # tiles handed out first come, first served (deterministic < 0) agree within the tolerance, not in every bit
    free_opt = yahkv.decode_options()
    free_opt.deterministic = -1
    free = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, opt=free_opt)
    assert rel_err(free, runs[0]) < 5e-4


@pytest.mark.parametrize("kind", ["bf16", "f32"])
def test_queries_beyond_the_f16_range_saturate(yahkv, torch_gpu, kind):
    """The kernels compute with f16 queries. A bf16 or f32 query element of 1e6 is taken as 65504 (not as infinity,
    which would turn its whole row into NaN); the result is the closed form of the saturated query."""
    torch = torch_gpu
    lens = [300, 70]
    g, table, host, dev, rng = setup(yahkv, torch, 8, 8, 2, 128, 16, lens, seed=77)
    q = to_bf16_f32(rng.standard_normal((2, 8, 128)))
    q[0, 3, 5], q[1, 0, 100] = 1e6, -3e38
    q = to_bf16_f32(q)
    got = gpu_attend(yahkv, torch, dev, table, lens, q, 1e-6, kind=kind)
    assert np.all(np.isfinite(got))
    sat = np.clip(q, -65504, 65504)
    assert rel_err(got, closed(g, table, host, lens, sat, 1e-6)) < TOL


def test_f32_queries_round_to_f16(yahkv, torch_gpu):
    """f32 queries (the reference's kernels take f32, gen_decode_attn.py:576-590) are rounded to f16, nearest even:
    the result is the closed form of the rounded query to well within the tolerance, and within it of the unrounded."""
    torch = torch_gpu
    lens = [513, 64]
    g, table, host, dev, rng = setup(yahkv, torch, 8, 24, 4, 256, 64, lens, seed=78)
    q = rng.standard_normal((2, 24, 256)).astype(np.float32)
    got = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, kind="f32")
    q16 = q.astype(np.float16).astype(np.float32)
    assert rel_err(got, closed(g, table, host, lens, q16, 0.0625)) < 5e-4
    assert rel_err(got, closed(g, table, host, lens, q, 0.0625)) < TOL


def test_xcd_calibration_returns_usable_shares(yahkv, torch_gpu):
    torch = torch_gpu
    rng0 = np.random.default_rng(5)
    lens = [int(x) for x in rng0.integers(2000, 30000, 48)]
    g, table, host, dev, rng = setup(yahkv, torch, 8, 24, 4, 256, 64, lens, seed=79)
    q = to_bf16_f32(rng.standard_normal((len(lens), 24, 256)))
    tq = torch.from_numpy(q).cuda().to(torch.bfloat16)
    t_table = torch.from_numpy(table).cuda()
    t_lens = torch.tensor(lens, dtype=torch.int32, device="cuda")
    opt = yahkv.decode_options()
    ws = torch.empty(yahkv.decode_workspace_bytes(g_dev(yahkv, g), len(lens), max(lens), opt), dtype=torch.uint8, device="cuda")
    w = yahkv.decode_calibrate(dev, t_table, t_lens, max(lens), tq, ws, opt, rounds=2)
    assert len(w) == 8 and max(w) == 10000 and min(w) >= 5000, w        # XCDs of one GPU lie within a few percent
    out = yahkv.decode_attend(dev, t_table, t_lens, max(lens), tq, 0.0625, workspace=ws, opt=opt)
    torch.cuda.synchronize()
    assert rel_err(out.cpu().numpy(), oracle.decode_attend(host, table, lens, q, 0.0625)) < TOL


def g_dev(yahkv, g):
    return yahkv.geometry(g.format, g.n_q_heads, g.n_kv_heads, g.head_dim, g.page_tokens, g.n_pages)


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt", [(8, 24, 4, 256, 64), (4, 24, 4, 256, 64), (8, 8, 2, 128, 16), (4, 16, 2, 256, 32)])
def test_one_launch_form_gives_the_two_dispatches_results(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt):
    """opt.one_launch: the workgroup that is last to finish a pair's keys merges the pair itself. Sequences that lie in
    one chunk, that span many, that are empty; on a workspace of random bytes that went through yahkv_decode_workspace_init
    once, twice in a row (the arrival counts of the first call are left at zero),
    then with the chunk count forced up so that every pair spans several chunks; with the deterministic pattern the
    one dispatch repeats bit for bit as well."""
    torch = torch_gpu
    lens = [1, 0, 63, 64, 65, 700, 5000, 31, 12000, 129, 2500, 0, 64 * 40]
    g, table, host, dev, rng = setup(yahkv, torch, fmt, n_q, n_kv, hd, pt, lens, seed=fmt + hd + pt, fill=0x7F)
    q = to_bf16_f32(rng.standard_normal((len(lens), n_q, hd)))
    gate = rng.standard_normal(q.shape).astype(np.float32)
    scale = float(1 / np.sqrt(hd))
    want = oracle.decode_attend(host, table, lens, q, scale, gate)
    for opt in (yahkv.decode_options(one_launch=True), yahkv.decode_options(one_launch=True, n_chunks=1000, min_chunk_tiles=2),
                yahkv.decode_options(one_launch=True, n_chunks=7)):
        ws = torch.empty(yahkv.decode_workspace_bytes(g_dev(yahkv, g), len(lens), max(lens), opt), dtype=torch.uint8, device="cuda")
        ws.random_(0, 256)                                     # junk everywhere, the arrival counts included ...
        yahkv.decode_workspace_init(g_dev(yahkv, g), len(lens), max(lens), ws, opt)   # ... which this call zeroes, once
        tq = torch.from_numpy(q).cuda().to(torch.bfloat16)
        tg = torch.from_numpy(gate).cuda()
        t_table = torch.from_numpy(table).cuda()
        t_lens = torch.tensor(lens, dtype=torch.int32, device="cuda")
        for _ in range(2):
            out = torch.full(q.shape, float("nan"), device="cuda")
            yahkv.decode_attend(dev, t_table, t_lens, max(lens), tq, scale, gate=tg, out=out, workspace=ws, opt=opt)
            torch.cuda.synchronize()
            got = out.cpu().numpy()
            assert np.all(np.isfinite(got))
            assert not got[1].any() and not got[11].any()
            assert rel_err(got, want) < TOL
    det = yahkv.decode_options(one_launch=True, deterministic=True)
    runs = [gpu_attend(yahkv, torch, dev, table, lens, q, scale, opt=det) for _ in range(3)]
    assert np.array_equal(runs[0].view(np.uint32), runs[1].view(np.uint32))
    assert np.array_equal(runs[0].view(np.uint32), runs[2].view(np.uint32))


@pytest.mark.parametrize("fmt,n_q,n_kv", [(8, 24, 4), (4, 16, 2), (8, 24, 8), (8, 18, 3)])
def test_cut_by_tile_and_by_head_agree(yahkv, torch_gpu, fmt, n_q, n_kv):
    """opt.cut: by (sequence, tile) with the kv heads of a tile on neighbouring waves (the default where the head count
    divides 8) and by (sequence, kv head) give the oracle's result, each bit for bit the same on a second call; with
    three kv heads both are the cut by head. Ragged lengths incl. empty and one-key sequences, with a gate; then the
    step form, pools byte for byte."""
    torch = torch_gpu
    lens = [1, 0, 63, 64, 65, 700, 5000, 31, 12000, 129, 2500, 0, 64 * 40, 33000]
    g, table, host, dev, rng = setup(yahkv, torch, fmt, n_q, n_kv, 256, 64, lens, seed=fmt + n_kv, fill=0x3C)
    q = to_bf16_f32(rng.standard_normal((len(lens), n_q, 256)))
    gate = rng.standard_normal(q.shape).astype(np.float32)
    want = oracle.decode_attend(host, table, lens, q, 0.0625, gate)
    outs = {}
    for cut in (1, 2, 0):
        opt = yahkv.decode_options(cut=cut)
        a = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, opt=opt, gate=gate)
        b = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, opt=opt, gate=gate)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), cut
        assert rel_err(a, want) < TOL, cut
        assert not a[1].any() and not a[11].any()
        outs[cut] = a
    assert np.array_equal(outs[0].view(np.uint32), outs[2 if 8 % n_kv == 0 else 1].view(np.uint32))
    assert rel_err(outs[1], outs[2]) < 5e-4


@pytest.mark.parametrize("lens", [
    [32769],                                   # one long sequence: 513 tiles per kv head, chunks of nine tiles (a wave takes two)
    [32000],                                   # ... of eight: one tile per wave
    [1], [63], [65],
    [1, 0, 63, 64, 65, 700, 129, 0, 31],       # pairs that end inside a chunk: most waves' shares go to memory one by one
    [3000, 5, 2000, 0, 1, 4100, 64],
    [9000, 8000, 7000, 6000],                  # the largest batches the whole-tile instance takes (two tiles per wave)
    [(i * 37) % 500 + (i % 7 != 0) for i in range(100)],   # a hundred short sequences, some empty: many pairs per chunk, and
                                                           # the cut by the whole workgroup (more than 64 sequences)
])
def test_small_batches_whole_tiles(yahkv, torch_gpu, lens):
    """A batch small enough for about a tile per wave (q8_0, head_dim 256, 64-token pages) goes to the instance of the
    part kernel that asks for a wave's whole tile at once (opt.wg_partials = 0 picks it by the batch's size, 3 asks for
    it). It gives the oracle's result, the same bits on a second call, and agrees with the rotating instances
    (wg_partials = 1: one partial per workgroup, 2: one per wave) to rounding; with a gate."""
    torch = torch_gpu
    g, table, host, dev, rng = setup(yahkv, torch, 8, 24, 4, 256, 64, lens, seed=len(lens) + lens[0], fill=0x3C)
    q = to_bf16_f32(rng.standard_normal((len(lens), 24, 256)))
    gate = rng.standard_normal(q.shape).astype(np.float32)
    want = oracle.decode_attend(host, table, lens, q, 0.0625, gate)
    outs = {}
    for mode in (0, 3, 1, 2):
        opt = yahkv.decode_options(wg_partials=mode)
        a = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, opt=opt, gate=gate)
        b = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625, opt=opt, gate=gate)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), mode
        assert rel_err(a, want) < TOL, mode
        for s, n in enumerate(lens):
            assert n > 0 or not a[s].any()
        outs[mode] = a
    assert np.array_equal(outs[0].view(np.uint32), outs[3].view(np.uint32))
    assert rel_err(outs[3], outs[1]) < 5e-4 and rel_err(outs[3], outs[2]) < 5e-4
