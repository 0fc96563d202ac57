"""Randomized sweeps of the append (pool bytes bit-exact against the CPU oracle) and of the chunked-prefill attention
(2e-3 against the oracle that models bf16 operands): formats, head counts, head dims, page sizes, batch sizes,
ragged start positions and valid counts, source dtypes, value scales over four decades, both prefill paths."""
import numpy as np
import pytest

import oracle
from helpers import make_tables, rel_err, to_bf16_f32, to_f16_f32
from test_gpu_append import same_pools, torch_src
from test_gpu_prefill import build

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed", range(16))
def test_random_append_case(yahkv, torch_gpu, seed):
    torch = torch_gpu
    rng = np.random.default_rng(2000 + seed)
    fmt = int(rng.choice([8, 4]))
    n_kv = int(rng.choice([1, 2, 4, 8]))
    hd = int(rng.choice([128, 256]))
    pt = int(rng.choice([16, 32, 64]))
    kind = str(rng.choice(["f32", "f16", "bf16"]))
    n_seqs = int(rng.integers(1, 9))
    rounds = int(rng.integers(1, 4))
    n_new = [int(rng.choice([1, 1, 7, 40, 129])) for _ in range(rounds)]
    pages = [(sum(n_new) + pt - 1) // pt + 1 for _ in range(n_seqs)]
    g = oracle.geometry(fmt, n_kv, n_kv, hd, pt, sum(pages) + 2)
    table = make_tables(rng, pages, g.n_pages)
    host = oracle.HostPools(g, fill=0x5A)
    dev = yahkv.DevicePools(yahkv.geometry(fmt, n_kv, n_kv, hd, pt, g.n_pages), fill=0x5A)
    t_table = torch.from_numpy(table).cuda()
    rnd = {"f32": lambda x: x.astype(np.float32), "f16": to_f16_f32, "bf16": to_bf16_f32}[kind]
    lens = np.zeros(n_seqs, np.int32)
    for n in n_new:
        valid = rng.integers(0, n + 1, n_seqs).astype(np.int32) if n > 1 else np.ones(n_seqs, np.int32)
        K = rnd(rng.standard_normal((n_seqs, n, n_kv, hd)) * 10.0 ** rng.uniform(-2, 2, (n_seqs, n, n_kv, 1)))
        V = rnd(rng.standard_normal((n_seqs, n, n_kv, hd)))
        if rng.random() < 0.3:
            K[:, :, :, : 32] = 0.0                               # all-zero blocks: scale 0, codes 0
        oracle.append(host, table, lens, valid, K, V)
        yahkv.append(dev, t_table, torch.from_numpy(lens.copy()).cuda(), torch_src(torch, K, kind),
                     torch_src(torch, V, kind), n_valid=torch.from_numpy(valid).cuda())
        lens = lens + valid
    same_pools(dev, host)                                        # written bytes equal, untouched bytes still 0x5A


@pytest.mark.parametrize("seed", range(10))
def test_random_prefill_case(yahkv, torch_gpu, seed):
    torch = torch_gpu
    rng = np.random.default_rng(3000 + seed)
    fmt = int(rng.choice([8, 4]))
    n_kv = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 3, 4, 6, 8]))
    hd = int(rng.choice([128, 256]))
    pt = int(rng.choice([16, 32, 64]))
    n_seqs = int(rng.integers(1, 4))
    prefix = [int(x) for x in rng.integers(0, 400, n_seqs)]
    chunk = int(rng.choice([1, 9, 64, 70, 150]))
    path = None if rng.random() < 0.6 else False                 # with a workspace (tile images), or the one-pass kernel
    g, table, host, dev, t_table, rng2, to_t = build(yahkv, torch, fmt, n_kv * group, n_kv, hd, pt, prefix, chunk,
                                                     seed=seed, fill=0x7F)
    q = to_bf16_f32(rng.standard_normal((n_seqs, chunk, n_kv * group, hd)))
    gate = rng.standard_normal(q.shape).astype(np.float32) if rng.random() < 0.3 else None
    scale = float(1 / np.sqrt(hd))
    t_prefix = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    out = yahkv.prefill_attend(dev, t_table, t_prefix, max(prefix) + int(rng.integers(0, 50)), to_t(q), scale,
                               gate=None if gate is None else torch.from_numpy(gate).cuda(), workspace=path)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got)), (fmt, n_kv, group, hd, pt, prefix, chunk, path)
    want = oracle.prefill_attend(host, table, prefix, q, scale, gate)
    assert rel_err(got, want) < 2e-3, (fmt, n_kv, group, hd, pt, prefix, chunk, path)
