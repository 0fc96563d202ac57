"""yahkv_decode_step: the append of a step's token and the attention over it in two dispatches. Held to what the two
separate calls give: the pools byte for byte (against the oracle's append, poison in every byte nobody writes), the
output within 2e-3 of the oracle's attention over the pools after the append, and close to the output of
yahkv_append + yahkv_decode_attend on a second copy of the pools. Sequences with nothing but the new token, empty
sequences (left alone), tokens that open a page, both formats, the three source types, a gate, tuning options."""
import ctypes as C

import numpy as np
import pytest

import oracle
from helpers import bf16_bits, make_tables, rel_err, to_bf16_f32

pytestmark = pytest.mark.gpu
TOL = 2e-3


def to_dev(torch, x, kind):
    if kind == "bf16":
        return torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)
    if kind == "f16":
        return torch.from_numpy(x.astype(np.float16)).cuda()
    return torch.from_numpy(x.astype(np.float32)).cuda()


def rounded(x, kind):
    """x as the device will see it."""
    if kind == "bf16":
        return to_bf16_f32(x)
    if kind == "f16":
        return x.astype(np.float16).astype(np.float32)
    return x.astype(np.float32)


def build(yahkv, fmt, n_q, n_kv, hd, pt, lens, seed):
    """Pools that hold all but the last token of every sequence; pages for the whole of it."""
    rng = np.random.default_rng(seed)
    pages = [(n + pt - 1) // pt for n in lens]
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, max(sum(pages), 1) + 2)
    table = make_tables(rng, pages, g.n_pages, stride=max(max(pages), 1))
    host = oracle.HostPools(g, fill=0x7F)
    for s, n in enumerate(lens):
        if n > 1:
            oracle.append(host, table[s:s + 1], [0], None, to_bf16_f32(rng.standard_normal((1, n - 1, n_kv, hd))),
                          to_bf16_f32(rng.standard_normal((1, n - 1, n_kv, hd))))
    devs = []
    for _ in range(2):
        dev = yahkv.DevicePools(yahkv.geometry(fmt, n_q, n_kv, hd, pt, g.n_pages))
        dev.load(host.arrays())
        devs.append(dev)
    return g, table, host, devs, rng


def run_case(yahkv, torch, fmt, n_q, n_kv, hd, pt, lens, seed, kind="bf16", qkind="bf16", gate=False, opt=None,
             slack=0):
    g, table, host, (dev, dev2), rng = build(yahkv, fmt, n_q, n_kv, hd, pt, lens, seed)
    B = len(lens)
    k_new = rounded(rng.standard_normal((B, n_kv, hd)) * 1.5, kind)
    v_new = rounded(rng.standard_normal((B, n_kv, hd)), kind)
    q = rounded(rng.standard_normal((B, n_q, hd)), qkind)
    gt = rng.standard_normal(q.shape).astype(np.float32) if gate else None
    scale = float(1 / np.sqrt(hd))
    for s, n in enumerate(lens):                         # what the step must leave in the pools
        if n >= 1:
            oracle.append(host, table[s:s + 1], [n - 1], None, k_new[s][None, None], v_new[s][None, None])
    want = oracle.decode_attend(host, table, lens, q, scale, gt)
    t_table = torch.from_numpy(table).cuda()
    t_lens = torch.tensor(lens, dtype=torch.int32, device="cuda")
    max_len = min(max(max(lens), 1) + slack, table.shape[1] * pt)
    tg = None if gt is None else torch.from_numpy(gt).cuda()
    tk, tv, tq = to_dev(torch, k_new, kind), to_dev(torch, v_new, kind), to_dev(torch, q, qkind)
    got = yahkv.decode_step(dev, t_table, t_lens, max_len, tk, tv, tq, scale, gate=tg, opt=opt)
    torch.cuda.synchronize()
    got = got.cpu().numpy()
    pools = dev.numpy()
    for name, arr in host.arrays().items():
        assert np.array_equal(pools[name], arr), f"pool {name}: the step's token or untouched bytes differ"
    assert np.all(np.isfinite(got))
    for s, n in enumerate(lens):
        if n == 0:
            assert not got[s].any(), "an empty sequence attends to nothing"
    assert rel_err(got, want) < TOL, (fmt, n_q, n_kv, hd, pt, lens)
    # the two separate calls on the second copy (append takes every sequence: give the empty ones n_valid = 0)
    live = torch.tensor([1 if n >= 1 else 0 for n in lens], dtype=torch.int32, device="cuda")
    yahkv.append(dev2, t_table, torch.clamp(t_lens - 1, min=0), tk[:, None], tv[:, None], n_valid=live)
    two = yahkv.decode_attend(dev2, t_table, t_lens, max_len, tq, scale, gate=tg, opt=opt).cpu().numpy()
    pools2 = dev2.numpy()
    for name in pools:
        assert np.array_equal(pools[name], pools2[name]), name
    # (the split-K kernel feeds the matrix unit V values rounded to f16, 2^-11 relative at most; the step's own token
    # enters the sums unrounded)
    assert rel_err(got, two) < 6e-4
    return got


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt,lens", [
    (8, 24, 4, 256, 64, [1, 2, 64, 65, 129, 700, 0, 1000]),
    (4, 24, 4, 256, 64, [1, 2, 64, 65, 129, 700, 0, 1000]),
    (8, 8, 2, 128, 16, [513, 17, 16, 1, 0, 33]),
    (4, 8, 2, 128, 16, [513, 17, 16, 1, 0, 33]),
    (8, 6, 2, 256, 32, [33, 32, 300]),
    (4, 16, 2, 128, 32, [97, 1, 1, 64]),
    (8, 4, 4, 128, 64, [5000]),
    (8, 24, 4, 256, 64, [1]),
])
def test_step_equals_append_then_attend(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt, lens):
    run_case(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt, lens, seed=fmt + hd + pt + len(lens))


@pytest.mark.parametrize("kind,qkind", [("f32", "f32"), ("f16", "f16"), ("bf16", "f32"), ("f32", "bf16")])
def test_source_and_query_types(yahkv, torch_gpu, kind, qkind):
    run_case(yahkv, torch_gpu, 8, 12, 2, 128, 32, [70, 1, 200, 0, 31], seed=11, kind=kind, qkind=qkind, gate=True)
    run_case(yahkv, torch_gpu, 4, 12, 2, 256, 64, [70, 1, 200, 0, 31], seed=12, kind=kind, qkind=qkind)


@pytest.mark.parametrize("seed", range(8))
def test_random_step(yahkv, torch_gpu, seed):
    rng = np.random.default_rng(4000 + seed)
    fmt = int(rng.choice([8, 4]))
    n_kv = int(rng.choice([1, 2, 4]))
    group = int(rng.choice([1, 2, 3, 4, 6, 8]))
    hd = int(rng.choice([128, 256]))
    pt = int(rng.choice([16, 32, 64]))
    lens = [int(x) for x in rng.integers(0, int(rng.choice([3, 70, 600])) + 1, int(rng.integers(1, 20)))]
    if max(lens) == 0:
        lens[0] = 1
    opt = yahkv.decode_options(n_chunks=int(rng.choice([0, 3, 13, 256])))
    opt.deterministic = int(rng.random() < 0.3)
    opt.reduce_split = int(rng.choice([0, 1, 2, 4]))
    run_case(yahkv, torch_gpu, fmt, n_kv * group, n_kv, hd, pt, lens, seed=seed, gate=bool(rng.random() < 0.3), opt=opt,
             slack=int(rng.integers(0, 50)))


def test_deterministic_step_repeats_its_bits(yahkv, torch_gpu):
    opt = yahkv.decode_options()
    opt.deterministic = 1
    a = run_case(yahkv, torch_gpu, 8, 24, 4, 256, 64, [3000, 1, 517], seed=21, opt=opt)
    b = run_case(yahkv, torch_gpu, 8, 24, 4, 256, 64, [3000, 1, 517], seed=21, opt=opt)
    assert np.array_equal(a, b)


def test_step_refuses_bad_arguments(yahkv, torch_gpu):
    torch = torch_gpu
    g = yahkv.geometry(8, 8, 2, 128, 16, 4)
    dev = yahkv.DevicePools(g)
    st = dev.struct()
    table = torch.zeros((1, 2), dtype=torch.int32, device="cuda")
    lens = torch.ones(1, dtype=torch.int32, device="cuda")
    kv = torch.zeros((1, 2, 128), dtype=torch.float32, device="cuda")
    q = torch.zeros((1, 8, 128), dtype=torch.float32, device="cuda")
    out = torch.zeros((1, 8, 128), dtype=torch.float32, device="cuda")
    ws = torch.empty(yahkv.decode_workspace_bytes(g, 1, 32), dtype=torch.uint8, device="cuda")

    def call(k=kv, v=kv, dtype=0, opt=None, o=out):
        return yahkv.lib.yahkv_decode_step(C.byref(g), C.byref(st), table.data_ptr(), 2, lens.data_ptr(), 1, 32,
                                           None if k is None else k.data_ptr(), None if v is None else v.data_ptr(),
                                           dtype, q.data_ptr(), 0, 0.1, None, None if o is None else o.data_ptr(),
                                           ws.data_ptr(), ws.numel(), opt, None)

    assert call() == 0
    torch.cuda.synchronize()
    assert call(k=None) == -1 and call(v=None) == -1 and call(o=None) == -1
    assert call(dtype=7) == -1
    one = yahkv.decode_options()
    one.one_launch = 1
    assert call(opt=C.byref(one)) == -1
    assert yahkv.lib.yahkv_decode_step(C.byref(g), C.byref(st), table.data_ptr(), 2, lens.data_ptr(), 1, 32,
                                       kv.data_ptr(), kv.data_ptr(), 0, q.data_ptr(), 0, 0.1, None, out.data_ptr(),
                                       ws.data_ptr(), 16, None, None) == -4


def test_large_batch_of_short_sequences_through_the_step(yahkv, torch_gpu):
    """1200 sequences of 0 to 40 tokens: most chunks span dozens of (sequence, kv head) pairs, many sequences have
    nothing but their new token (no partial at all), some have none."""
    rng = np.random.default_rng(91)
    lens = [int(x) for x in rng.integers(0, 41, 1200)]
    run_case(yahkv, torch_gpu, 8, 8, 2, 128, 16, lens, seed=92)


def test_positions_past_the_table_clamp_as_in_the_append(yahkv, torch_gpu):
    """Lengths that the host's validation would refuse still behave as the two separate calls do. A length beyond what
    the page table covers: the token goes to the table's last slot, as yahkv_append puts it (positions clamp to the
    table, gen_decode_attn.py:59-63), and the attention runs over the table's extent. A length beyond the host's bound
    where the table reaches further: the token is stored at its position and the attention stops short of it."""
    torch = torch_gpu
    rng = np.random.default_rng(93)
    n_q, n_kv, hd, pt = 8, 2, 128, 16
    g, table, host, (dev, dev2), _ = build(yahkv, 8, n_q, n_kv, hd, pt, [49, 49, 49], seed=94)   # 48 tokens held each
    table = table[:, :3].copy()                           # ... and a table that ends there
    extent = table.shape[1] * pt
    t_table = torch.from_numpy(table).cuda()
    k = to_dev(torch, to_bf16_f32(rng.standard_normal((3, n_kv, hd))), "bf16")
    v = to_dev(torch, to_bf16_f32(rng.standard_normal((3, n_kv, hd))), "bf16")
    q = to_dev(torch, to_bf16_f32(rng.standard_normal((3, n_q, hd))), "bf16")
    for lens, bound in (([extent + 7, extent, 20], extent + 7), ([40, 31, 30], 30)):
        t_lens = torch.tensor(lens, dtype=torch.int32, device="cuda")
        got = yahkv.decode_step(dev, t_table, t_lens, bound, k, v, q, 0.1).cpu().numpy()
        yahkv.append(dev2, t_table, t_lens - 1, k[:, None], v[:, None])
        two = yahkv.decode_attend(dev2, t_table, t_lens, bound, q, 0.1).cpu().numpy()
        a, b = dev.numpy(), dev2.numpy()
        for name in a:
            assert np.array_equal(a[name], b[name]), (name, lens)
        assert np.all(np.isfinite(got)) and rel_err(got, two) < 6e-4, lens
