"""Randomized sweep of the paged decode attention against the CPU oracle: formats, group sizes, head dims, page sizes,
batch sizes, ragged lengths with empty sequences, query dtypes, a gate now and then, and the planner's chunk count
forced to values that are not a multiple of eight, smaller than the work and larger than it. Tolerance 2e-3."""
import numpy as np
import pytest

import oracle
from helpers import rel_err, to_bf16_f32
from test_gpu_decode import gpu_attend, setup

pytestmark = pytest.mark.gpu
TOL = 2e-3


@pytest.mark.parametrize("seed", range(20))
def test_random_decode_case(yahkv, torch_gpu, seed):
    rng = np.random.default_rng(1000 + seed)
    fmt = int(rng.choice([8, 4]))
    n_kv = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 3, 4, 6, 8]))
    hd = int(rng.choice([128, 256]))
    pt = int(rng.choice([16, 32, 64]))
    n_seqs = int(rng.integers(1, 24))
    top = int(rng.choice([70, 300, 900]))
    lens = [int(x) for x in rng.integers(0, top + 1, n_seqs)]
    if rng.random() < 0.5:
        lens[int(rng.integers(0, n_seqs))] = 0               # an empty sequence in the batch
    if max(lens) == 0:
        lens[0] = 1
    chunks = int(rng.choice([0, 1, 3, 7, 13, 64, 100, 256, 1000]))
    opt = yahkv.decode_options(n_chunks=chunks)
    if rng.random() < 0.3:
        opt.min_chunk_tiles = int(rng.choice([1, 2, 5]))
    if rng.random() < 0.3:
        opt.deterministic = 1
    if rng.random() < 0.5:
        opt.one_launch = 1
    if rng.random() < 0.3:
        for j in range(8):
            opt.xcd_weight[j] = int(rng.choice([0, 1, 900, 1000, 1100, 100000]))
    g, table, host, dev, _ = setup(yahkv, torch_gpu, fmt, n_kv * group, n_kv, hd, pt, lens, seed=seed, fill=0x7F)
    q = to_bf16_f32(rng.standard_normal((n_seqs, n_kv * group, hd)))
    gate = rng.standard_normal(q.shape).astype(np.float32) if rng.random() < 0.3 else None
    kind = str(rng.choice(["bf16", "f16", "f32"]))
    if kind == "f16":
        q = q.astype(np.float16).astype(np.float32)
    scale = float(1 / np.sqrt(hd))
    slack = int(rng.integers(0, 100))                          # the host's bound may be loose
    got = gpu_attend(yahkv, torch_gpu, dev, table, lens, q, scale, gate=gate, kind=kind,
                     max_len=min(max(lens) + slack, table.shape[1] * pt), opt=opt)
    want = oracle.decode_attend(host, table, lens, q, scale, gate)
    assert np.all(np.isfinite(got)), (fmt, n_kv, group, hd, pt, lens, chunks)
    for s, n in enumerate(lens):
        if n == 0:
            assert not got[s].any(), "an empty sequence attends to nothing"
    assert rel_err(got, want) < TOL, (fmt, n_kv, group, hd, pt, lens, chunks, kind)


def test_large_batch_of_short_sequences(yahkv, torch_gpu):
    """1500 sequences of 0 to 40 tokens: every thread of a workgroup owns several sequences when the chunk records are
    computed, chunks span dozens of (sequence, kv head) pairs, and most partial slots stay empty."""
    rng = np.random.default_rng(77)
    n_seqs, n_kv, group, hd, pt = 1500, 2, 4, 128, 16
    lens = [int(x) for x in rng.integers(0, 41, n_seqs)]
    g, table, host, dev, _ = setup(yahkv, torch_gpu, 8, n_kv * group, n_kv, hd, pt, lens, seed=78, fill=0x7F)
    q = to_bf16_f32(rng.standard_normal((n_seqs, n_kv * group, hd)))
    scale = float(1 / np.sqrt(hd))
    got = gpu_attend(yahkv, torch_gpu, dev, table, lens, q, scale)
    want = oracle.decode_attend(host, table, lens, q, scale)
    assert np.all(np.isfinite(got))
    assert rel_err(got, want) < TOL
    for s in np.flatnonzero(np.array(lens) == 0)[:20]:
        assert not got[s].any()


def test_chunks_of_one_or_two_units(yahkv, torch_gpu):
    """The finest cut the planner allows (asked for one tile per chunk; it keeps two line units): the eight chunks of
    a group then differ by whole units, and none inside a pair's stretch may come out empty, because the reduce reads
    the partials of every chunk between a pair's first and last."""
    rng = np.random.default_rng(239)
    lens = [91, 627, 798, 425, 27, 408, 417, 18, 247, 137, 144, 127, 70, 839, 137, 273]
    for fmt, pair_cost, weights in ((4, 8, None), (8, -1, None), (8, 3, None), (8, 8, [1, 100000, 1, 1, 50000, 1, 1, 1])):
        opt = yahkv.decode_options(n_chunks=1000, min_chunk_tiles=1, pair_cost=pair_cost, xcd_weight=weights)
        g, table, host, dev, _ = setup(yahkv, torch_gpu, fmt, 8, 2, 256, 64, lens, seed=239, fill=0x7F)
        q = to_bf16_f32(rng.standard_normal((len(lens), 8, 256)))
        got = gpu_attend(yahkv, torch_gpu, dev, table, lens, q, 0.0625, max_len=896, opt=opt)
        assert np.all(np.isfinite(got))
        assert rel_err(got, oracle.decode_attend(host, table, lens, q, 0.0625)) < TOL


def test_the_largest_batch_a_call_takes_and_one_more(yahkv, torch_gpu):
    """8191 sequences in one call (the limit) against the oracle; 8192 are refused as a shape this build has no
    kernel for, before anything is launched."""
    torch = torch_gpu
    rng = np.random.default_rng(79)
    n_seqs, n_kv, group, hd, pt = 8191, 1, 2, 128, 16
    lens = [int(x) for x in rng.integers(0, 21, n_seqs)]
    g, table, host, dev, _ = setup(yahkv, torch, 8, n_kv * group, n_kv, hd, pt, lens, seed=80, fill=0x7F)
    q = to_bf16_f32(rng.standard_normal((n_seqs, n_kv * group, hd)))
    scale = float(1 / np.sqrt(hd))
    got = gpu_attend(yahkv, torch, dev, table, lens, q, scale)
    want = oracle.decode_attend(host, table, lens, q, scale)
    assert np.all(np.isfinite(got))
    assert rel_err(got, want) < TOL
    more = np.concatenate([table, table[:1]])
    with pytest.raises(yahkv.YahkvError) as e:
        gpu_attend(yahkv, torch, dev, more, lens + [1], np.concatenate([q, q[:1]]), scale)
    assert e.value.status == -2
