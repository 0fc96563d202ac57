"""GPU paged decode attention against the CPU oracle and the float64 closed form (tolerance 2e-3 max relative error,
max |got - want| / max |want|, the reference checker's metric), through the C ABI."""
import numpy as np
import pytest

import oracle
from helpers import bf16_bits, closed_form, dequant, logical_blocks, make_tables, rel_err, to_bf16_f32, to_f16_f32

pytestmark = pytest.mark.gpu
TOL = 2e-3


def setup(yahkv, torch, fmt, n_q, n_kv, hd, pt, lens, seed, extra_pages=2, fill=0):
    """Pools filled on the host by the oracle, uploaded as they are."""
    rng = np.random.default_rng(seed)
    pages = [(n + pt - 1) // pt for n in lens]
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, max(sum(pages), 1) + extra_pages)
    table = make_tables(rng, pages, g.n_pages, stride=max(max(pages), 1))
    host = oracle.HostPools(g, fill=fill)
    for s, n in enumerate(lens):
        if n:
            oracle.append(host, table[s:s + 1], [0], None, to_bf16_f32(rng.standard_normal((1, n, n_kv, hd))),
                          to_bf16_f32(rng.standard_normal((1, n, n_kv, hd))))
    dev = yahkv.DevicePools(yahkv.geometry(fmt, n_q, n_kv, hd, pt, g.n_pages))
    dev.load(host.arrays())
    return g, table, host, dev, rng


def gpu_attend(yahkv, torch, dev, table, lens, q, scale, gate=None, kind="bf16", max_len=None, opt=None):
    if kind == "bf16":
        tq = torch.from_numpy(bf16_bits(q).view(np.int16)).cuda().view(torch.bfloat16)
    elif kind == "f16":
        tq = torch.from_numpy(q.astype(np.float16)).cuda()
    else:
        tq = torch.from_numpy(q.astype(np.float32)).cuda()
    tg = None if gate is None else torch.from_numpy(gate.astype(np.float32)).cuda()
    out = yahkv.decode_attend(dev, torch.from_numpy(table).cuda(), torch.tensor(lens, dtype=torch.int32, device="cuda"),
                              max_len or max(max(lens), 1), tq, scale, gate=tg, opt=opt)
    torch.cuda.synchronize()
    return out.cpu().numpy()


def closed(g, table, host, lens, q, scale, gate=None):
    want = np.zeros(q.shape)
    for s, n in enumerate(lens):
        if n == 0:
            continue
        (ks, kc), (vs, vc) = logical_blocks(host.arrays(), g, table[s], n)
        want[s] = closed_form(dequant(ks, kc), dequant(vs, vc), q[s], scale, None if gate is None else gate[s])
    return want


def test_config1_tiny(yahkv, torch_gpu):
    """8 Q / 2 KV heads, head_dim 128, 16-token pages, 512-token prefix + 1 appended token, fp16 query."""
    torch = torch_gpu
    rng = np.random.default_rng(1)
    g = oracle.geometry(8, 8, 2, 128, 16, 33)
    K = to_f16_f32(rng.standard_normal((1, 513, 2, 128)))
    V = to_f16_f32(rng.standard_normal((1, 513, 2, 128)))
    table = np.random.default_rng(2).permutation(33).astype(np.int32)[None]
    q = to_f16_f32(np.random.default_rng(3).standard_normal((1, 8, 128)))
    host = oracle.HostPools(g)
    oracle.append(host, table, [0], None, K, V)
    dev = yahkv.DevicePools(yahkv.geometry(8, 8, 2, 128, 16, 33))
    t_table = torch.from_numpy(table).cuda()
    pos = torch.zeros(1, dtype=torch.int32, device="cuda")
    yahkv.append(dev, t_table, pos, torch.from_numpy(K[:, :512].astype(np.float16)).cuda(),
                 torch.from_numpy(V[:, :512].astype(np.float16)).cuda())
    yahkv.append(dev, t_table, pos + 512, torch.from_numpy(K[:, 512:].astype(np.float16)).cuda(),
                 torch.from_numpy(V[:, 512:].astype(np.float16)).cuda())
    got_pools = dev.numpy()
    for name, want in host.arrays().items():
        assert np.array_equal(got_pools[name], want), name
    scale = 1 / np.sqrt(128)
    got = gpu_attend(yahkv, torch, dev, table, [513], q, scale, kind="f16")
    assert rel_err(got, oracle.decode_attend(host, table, [513], q, scale)) < TOL
    assert rel_err(got, closed(g, table, host, [513], q, scale)) < TOL
    prev = gpu_attend(yahkv, torch, dev, table, [512], q, scale, kind="f16")
    assert rel_err(prev, closed(g, table, host, [512], q, scale)) < TOL
    assert np.abs(prev - got).max() > 1e-6          # the appended token is visible only from its own step on


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt", [(8, 24, 4, 256, 64), (4, 24, 4, 256, 64), (8, 8, 2, 128, 16),
                                                 (4, 8, 2, 128, 16), (8, 8, 1, 256, 32), (8, 4, 4, 128, 64), (8, 16, 2, 256, 16),
                                                 (8, 24, 4, 128, 32), (4, 8, 1, 256, 32), (4, 16, 2, 256, 16),
                                                 (4, 24, 4, 128, 32), (4, 4, 4, 128, 64)])
def test_ragged_batch_with_gate(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt):
    torch = torch_gpu
    lens = [1, pt - 1, pt, pt + 1, 63, 64, 65, 5 * 64 + 17, 1500, 0, 257]
    g, table, host, dev, rng = setup(yahkv, torch, fmt, n_q, n_kv, hd, pt, lens, seed=fmt * 1000 + hd + pt, fill=0x7C)
    q = to_bf16_f32(rng.standard_normal((len(lens), n_q, hd)))
    gate = rng.standard_normal((len(lens), n_q, hd)).astype(np.float32)
    scale = 1 / np.sqrt(hd)
    for gt in (None, gate):
        got = gpu_attend(yahkv, torch, dev, table, lens, q, scale, gt)
        assert np.all(np.isfinite(got))
        assert np.all(got[lens.index(0)] == 0)
        assert rel_err(got, oracle.decode_attend(host, table, lens, q, scale, gt)) < TOL
        want = closed(g, table, host, lens, q, scale, gt)
        for s in range(len(lens)):
            if lens[s]:
                assert rel_err(got[s], want[s]) < TOL, (s, lens[s])


def test_special_cases(yahkv, torch_gpu):
    torch = torch_gpu
    lens = [1, 200]
    g, table, host, dev, rng = setup(yahkv, torch, 8, 24, 4, 256, 64, lens, seed=9, fill=0xFF)
    (_, _), (vs, vc) = logical_blocks(host.arrays(), g, table[0], 1)
    q = to_bf16_f32(rng.standard_normal((2, 24, 256)))
    out = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625)
    assert rel_err(out[0], np.repeat(dequant(vs, vc)[0], 6, 0)) < 1e-3          # one key: its V row
    out = gpu_attend(yahkv, torch, dev, table, lens, np.zeros_like(q), 0.0625)
    (ks, kc), (vs, vc) = logical_blocks(host.arrays(), g, table[1], 200)
    Kd, Vd = dequant(ks, kc), dequant(vs, vc)
    assert rel_err(out[1], np.repeat(Vd.mean(0), 6, 0)) < 1e-3                   # equal scores: the mean of V
    q[1, 1] = q[1, 0]
    out = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625)
    assert np.array_equal(out[1, 0], out[1, 1])                                  # same query, same GQA group
    q[1, 7] = to_bf16_f32(60 * Kd[117, 1] / np.linalg.norm(Kd[117, 1]))
    out = gpu_attend(yahkv, torch, dev, table, lens, q, 1.0)
    assert np.abs(out[1, 7] - Vd[117, 1]).max() < 2e-3 * np.abs(Vd[117, 1]).max()   # one huge score: that V row


@pytest.mark.parametrize("fmt", [8, 4])
def test_stale_bytes_past_the_length_are_masked(yahkv, torch_gpu, fmt):
    """Slots past seq_len hold poison (NaN scales, 0x7F codes): they must not reach the output."""
    torch = torch_gpu
    lens = [70, 3]
    g, table, host, dev, rng = setup(yahkv, torch, fmt, 24, 4, 256, 64, lens, seed=10, fill=0x7F)  # f16 0x7F7F is NaN
    q = to_bf16_f32(rng.standard_normal((2, 24, 256)))
    got = gpu_attend(yahkv, torch, dev, table, lens, q, 0.0625)
    assert np.all(np.isfinite(got))
    assert rel_err(got, closed(g, table, host, lens, q, 0.0625)) < TOL


def test_lengths_are_clamped_to_max_seq_len_and_table(yahkv, torch_gpu):
    torch = torch_gpu
    lens = [300, 40]
    g, table, host, dev, rng = setup(yahkv, torch, 8, 8, 2, 128, 16, lens, seed=11)
    q = to_bf16_f32(rng.standard_normal((2, 8, 128)))
    got = gpu_attend(yahkv, torch, dev, table, [10 ** 6, 40], q, 0.09, max_len=300)
    want = closed(g, table, host, [300, 40], q, 0.09)
    assert rel_err(got, want) < TOL


def test_workspace_and_argument_checks(yahkv, torch_gpu):
    import ctypes as C
    torch = torch_gpu
    g = yahkv.geometry(8, 24, 4, 256, 64, 8)
    dev = yahkv.DevicePools(g)
    need = yahkv.decode_workspace_bytes(g, 2, 300)
    assert need > 0
    # the workspace's size follows the options: both calls must be given the same ones
    assert yahkv.decode_workspace_bytes(g, 2, 300, yahkv.decode_options(n_chunks=8, min_chunk_tiles=2)) != need
    table = torch.zeros((2, 5), dtype=torch.int32, device="cuda")
    lens = torch.tensor([5, 6], dtype=torch.int32, device="cuda")
    q = torch.zeros((2, 24, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(yahkv.YahkvError) as e:
        yahkv.decode_attend(dev, table, lens, 300, q, 0.0625, workspace=torch.empty(need - 16, dtype=torch.uint8, device="cuda"))
    assert e.value.status == -4
    st = dev.struct()
    rc = yahkv.lib.yahkv_decode_attend(C.byref(g), C.byref(st), None, 5, None, 2, 300, None, 2, 0.0625, None, None, None, 0,
                                       None, None)
    assert rc == -1
