"""GPU chunked-prefill attention against the CPU oracle's exact arithmetic on the dequantized K / V (f64 sums, nothing
of the matrix unit's operand rounding modelled): tolerance 2e-3 max relative error, max |got - want| / max |want|. The
kernels feed the matrix unit f16 keys, values and numerators (2^-12 relative each); measured 2e-4 .. 5e-4."""
import numpy as np
import pytest

import oracle
from helpers import bf16_bits, closed_form, dequant, logical_blocks, make_tables, rel_err, to_bf16_f32

pytestmark = pytest.mark.gpu
TOL = 2e-3


def build(yahkv, torch, fmt, n_q, n_kv, hd, pt, prefix, chunk, seed, fill=0):
    rng = np.random.default_rng(seed)
    lens = [p + chunk for p in prefix]
    pages = [(n + pt - 1) // pt for n in lens]
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, sum(pages) + 2)
    table = make_tables(rng, pages, g.n_pages)
    host = oracle.HostPools(g, fill=fill)
    dev = yahkv.DevicePools(yahkv.geometry(fmt, n_q, n_kv, hd, pt, g.n_pages), fill=fill)
    t_table = torch.from_numpy(table).cuda()
    to_t = lambda x: torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)
    for s, p in enumerate(prefix):                       # the prefix, then the chunk, both through the GPU append
        for start, n in ((0, p), (p, chunk)):
            if n == 0:
                continue
            k = to_bf16_f32(rng.standard_normal((1, n, n_kv, hd)))
            v = to_bf16_f32(rng.standard_normal((1, n, n_kv, hd)))
            oracle.append(host, table[s:s + 1], [start], None, k, v)
            yahkv.append(dev, t_table[s:s + 1], torch.tensor([start], dtype=torch.int32, device="cuda"), to_t(k), to_t(v))
    got = dev.numpy()
    for name, want in host.arrays().items():
        assert np.array_equal(got[name], want), name
    return g, table, host, dev, t_table, rng, to_t


# path "images": decode to f16 tile images in a workspace, then attention; "fused": one kernel, no workspace
@pytest.mark.parametrize("path,fmt,n_q,n_kv,hd,pt,prefix,chunk", [
    ("images", 8, 24, 4, 256, 64, [100, 0, 64 * 3 + 5], 70),
    ("images", 8, 24, 4, 256, 64, [1000], 256),
    ("images", 8, 8, 2, 128, 16, [37, 0, 64], 21),
    ("images", 8, 6, 2, 256, 32, [31, 500], 64),
    ("images", 8, 10, 2, 128, 64, [129], 130),
    ("images", 8, 12, 4, 128, 64, [70, 300], 100),
    ("images", 8, 6, 1, 128, 32, [1], 65),
    ("images", 4, 24, 4, 256, 64, [100, 0, 64 * 3 + 5], 70),
    ("images", 4, 8, 2, 128, 16, [37, 0, 64], 21),
    ("images", 4, 6, 2, 256, 32, [31, 500], 64),
    ("fused", 8, 24, 4, 256, 64, [100, 0, 64 * 3 + 5], 70),
    ("fused", 8, 24, 4, 256, 64, [1000], 256),
    ("fused", 8, 8, 2, 128, 16, [37, 0, 64], 21),
    ("fused", 8, 6, 2, 256, 32, [31, 500], 64),
    ("fused", 8, 10, 2, 128, 64, [129], 130),
    ("fused", 4, 24, 4, 256, 64, [100, 0, 64 * 3 + 5], 70),
    ("fused", 4, 8, 2, 128, 16, [37, 0, 64], 21),
    ("fused", 4, 6, 2, 256, 32, [31, 500], 64),
])
def test_prefill_against_oracle(yahkv, torch_gpu, path, fmt, n_q, n_kv, hd, pt, prefix, chunk):
    torch = torch_gpu
    ws = None if path == "images" else False
    g, table, host, dev, t_table, rng, to_t = build(yahkv, torch, fmt, n_q, n_kv, hd, pt, prefix, chunk,
                                                    seed=hd + pt + chunk, fill=0x7F)
    q = to_bf16_f32(rng.standard_normal((len(prefix), chunk, n_q, hd)))
    gate = rng.standard_normal(q.shape).astype(np.float32)
    scale = 1 / np.sqrt(hd)
    t_prefix = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    for gt in (None, gate):
        tg = None if gt is None else torch.from_numpy(gt).cuda()
        out = yahkv.prefill_attend(dev, t_table, t_prefix, max(prefix), to_t(q), scale, gate=tg, workspace=ws)
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        assert np.all(np.isfinite(got))
        exact = oracle.prefill_attend(host, table, prefix, q, scale, gt)
        assert rel_err(got, exact) < 1e-3                        # half the tolerance: measured 2e-4 .. 5e-4
    exact = oracle.prefill_attend(host, table, prefix, q, scale, None)
    # f16 output (what the reference's kernel writes, gen_attn_fa.py:1589-1595): the same numbers rounded once more
    out16 = yahkv.prefill_attend(dev, t_table, t_prefix, max(prefix), to_t(q), scale, out_dtype=torch.float16,
                                 workspace=ws)
    assert rel_err(out16.float().cpu().numpy(), exact) < TOL
    # bf16 output: its own rounding comes on top, up to 2^-8 of an element (8 significant bits), which is more than
    # the whole tolerance: callers that need 2e-3 take f16 or f32 output
    out16 = yahkv.prefill_attend(dev, t_table, t_prefix, max(prefix), to_t(q), scale, out_dtype=torch.bfloat16,
                                 workspace=ws)
    assert rel_err(out16.float().cpu().numpy(), exact) < 1e-3 + 2.0 ** -8


@pytest.mark.parametrize("ws", [None, False], ids=["images", "fused"])
def test_prefill_special_cases(yahkv, torch_gpu, ws):
    """Closed-form checks: the first query of a sequence without prefix returns its own V row; a chunk of one query
    equals decode attention at that length; independent float64 closed form for a few rows."""
    torch = torch_gpu
    prefix, chunk = [0, 77], 40
    g, table, host, dev, t_table, rng, to_t = build(yahkv, torch, 8, 24, 4, 256, 64, prefix, chunk, seed=5)
    q = to_bf16_f32(rng.standard_normal((2, chunk, 24, 256)))
    t_prefix = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    got = yahkv.prefill_attend(dev, t_table, t_prefix, 77, to_t(q), 0.0625, workspace=ws).cpu().numpy()
    (ks, kc), (vs, vc) = logical_blocks(host.arrays(), g, table[0], chunk)
    Kd, Vd = dequant(ks, kc), dequant(vs, vc)
    v16 = Vd[0].astype(np.float16).astype(np.float32)
    assert rel_err(got[0, 0], np.repeat(v16, 6, 0)) < 1e-6                       # one visible key: out = f16(V row)
    for t in (1, 17, chunk - 1):
        assert rel_err(got[0, t], closed_form(Kd[:t + 1], Vd[:t + 1], q[0, t], 0.0625)) < TOL
    lens = [p + chunk for p in prefix]
    one = yahkv.prefill_attend(dev, t_table, torch.tensor([l - 1 for l in lens], dtype=torch.int32, device="cuda"),
                               max(lens), to_t(q[:, -1:]), 0.0625, workspace=ws).cpu().numpy()
    dec = yahkv.decode_attend(dev, t_table, torch.tensor(lens, dtype=torch.int32, device="cuda"), max(lens),
                              to_t(q[:, -1]), 0.0625).cpu().numpy()
    assert rel_err(one[:, 0], dec) < TOL
    assert rel_err(one[:, 0], got[:, -1]) < 1e-6                                 # same query, same keys, same kernel


def test_both_paths_agree(yahkv, torch_gpu):
    """The two paths feed the matrix unit the same f16 values; only the order of the f32 sums differs."""
    torch = torch_gpu
    prefix, chunk = [300, 5], 100
    g, table, host, dev, t_table, rng, to_t = build(yahkv, torch, 8, 24, 4, 256, 64, prefix, chunk, seed=6)
    q = to_t(to_bf16_f32(rng.standard_normal((2, chunk, 24, 256))))
    t_prefix = torch.tensor(prefix, dtype=torch.int32, device="cuda")
    a = yahkv.prefill_attend(dev, t_table, t_prefix, 300, q, 0.0625).cpu().numpy()
    b = yahkv.prefill_attend(dev, t_table, t_prefix, 300, q, 0.0625, workspace=False).cpu().numpy()
    assert rel_err(a, b) < 2e-4
    ws = torch.empty(yahkv.prefill_workspace_bytes(dev.geom, 2, 400, chunk), dtype=torch.uint8, device="cuda")
    c = yahkv.prefill_attend(dev, t_table, t_prefix, 400, q, 0.0625, workspace=ws).cpu().numpy()   # a looser bound
    assert np.array_equal(a, c)


def test_prefill_rejects_bad_arguments(yahkv, torch_gpu):
    import ctypes as C
    torch = torch_gpu
    g = yahkv.geometry(4, 24, 4, 256, 64, 8)
    dev = yahkv.DevicePools(g)
    table = torch.zeros((1, 4), dtype=torch.int32, device="cuda")
    q = torch.zeros((1, 8, 24, 256), dtype=torch.bfloat16, device="cuda")
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    with pytest.raises(yahkv.YahkvError) as e:                                    # workspace too small
        yahkv.prefill_attend(dev, table, zero, 0, q, 0.0625, workspace=torch.empty(256, dtype=torch.uint8, device="cuda"))
    assert e.value.status == -4
    with pytest.raises(yahkv.YahkvError) as e:                                    # scale must be positive
        yahkv.prefill_attend(dev, table, zero, 0, q, 0.0)
    assert e.value.status == -1
    g8 = yahkv.geometry(8, 24, 4, 256, 64, 8)
    st = yahkv.DevicePools(g8).struct()
    rc = yahkv.lib.yahkv_prefill_attend(C.byref(g8), C.byref(st), None, 4, None, 1, 0, 8, None, 0.0625, None, None, 0,
                                        None, 0, None)
    assert rc == -1
    # a kv head's tile images beyond 2 GiB (prefix + chunk past 2^21 tokens at head_dim 256): refused as a shape, before
    # the workspace's size is even looked at (the size given is the buffer's real one: were the refusal missing, the
    # answer would be "workspace too small", never a launch)
    out = torch.empty(q.shape, dtype=torch.bfloat16, device="cuda")
    small = torch.empty(4096, dtype=torch.uint8, device="cuda")
    rc = yahkv.lib.yahkv_prefill_attend_tiles(C.byref(g8), C.byref(st), table.data_ptr(), 4, zero.data_ptr(), 1, 1 << 21, 8,
                                              q.data_ptr(), 0.0625, None, out.data_ptr(), 2, small.data_ptr(), 4096,
                                              None)
    assert rc == -2
