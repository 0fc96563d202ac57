"""The unquantized f16 twins of the decode path (yahkv_f16_append, yahkv_f16_decode_attend; the reference's
yah_dattn_kvappend / part / reduce, gen_decode_attn.py:30-411). Nothing of the quantized oracle applies: the append is
a conversion (pinned bit for bit by numpy's IEEE float16 rounding) and the attention is pinned by the float64 closed
form over the f16 values, within the 2e-3 of the quantized path."""
import numpy as np
import pytest

from helpers import bf16_bits, to_bf16_f32

pytestmark = pytest.mark.gpu


def tensor(torch, x, kind):
    if kind == "f32":
        return torch.from_numpy(np.ascontiguousarray(x, np.float32)).cuda()
    if kind == "f16":
        return torch.from_numpy(x.astype(np.float16)).cuda()
    return torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)


def gather(yahkv, dev, table_row, n):
    """Logical K and V [n][H][D] (float16) read back through one sequence's page-table row."""
    g = dev.geom
    k, v = dev.numpy()
    pt, d = g.page_tokens, g.head_dim
    K = np.zeros((n, g.n_kv_heads, d), np.float16)
    V = np.zeros((n, g.n_kv_heads, d), np.float16)
    for p in range(n):
        page, t = int(table_row[p // pt]), p % pt
        K[p] = k[page, :, :, t, :].reshape(g.n_kv_heads, d).view(np.float16)
        V[p] = v[page, :, :, t].view(np.float16)
    return K, V


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("hd,pt", [(128, 16), (256, 64), (256, 32)])
def test_append_is_the_f16_rounding_at_the_page_rows(yahkv, torch_gpu, kind, hd, pt):
    torch = torch_gpu
    rng = np.random.default_rng(hd + pt)
    n_kv, lens, chunk = 2, [37, 5, 0], 40
    pages = (max(lens) + chunk + pt - 1) // pt
    g = yahkv.f16_geometry(4, n_kv, hd, pt, 3 * pages)
    table = rng.permutation(3 * pages).astype(np.int32).reshape(3, pages)
    dev = yahkv.F16Pools(g, fill=0xAB)
    src_k = rng.standard_normal((3, chunk, n_kv, hd)).astype(np.float32) * 3.0
    src_v = rng.standard_normal((3, chunk, n_kv, hd)).astype(np.float32) * 70000.0  # some overflow f16: inf on both sides
    if kind == "bf16":
        src_k, src_v = to_bf16_f32(src_k), to_bf16_f32(src_v)
    if kind == "f16":
        src_k = src_k.astype(np.float16).astype(np.float32)
        src_v = np.clip(src_v, -60000, 60000).astype(np.float16).astype(np.float32)
    start = torch.tensor(lens, dtype=torch.int32, device="cuda")
    valid = torch.tensor([chunk, 7, 1], dtype=torch.int32, device="cuda")
    yahkv.f16_append(dev, torch.from_numpy(table).cuda(), start, tensor(torch, src_k, kind), tensor(torch, src_v, kind),
                     n_valid=valid)
    k, v = dev.numpy()
    written = np.zeros(k.shape[:2] + (pt,), bool)
    with np.errstate(over="ignore"):
        for s, (l0, nv) in enumerate(zip(lens, [chunk, 7, 1])):
            K, V = gather(yahkv, dev, table[s], l0 + nv)
            assert np.array_equal(K[l0:].view(np.uint16), src_k[s, :nv].astype(np.float16).view(np.uint16))
            assert np.array_equal(V[l0:].view(np.uint16), src_v[s, :nv].astype(np.float16).view(np.uint16))
            for p in range(l0, l0 + nv):
                written[table[s, p // pt], :, p % pt] = True
    # nothing else was touched
    assert np.all(k[~written[:, :, None, :].repeat(hd // 16, 2)] == 0xABAB)
    assert np.all(v[~written[:, :, None, :].repeat(hd, 2)] == 0xABAB)


def test_positions_clamp_and_the_last_token_wins(yahkv, torch_gpu):
    torch = torch_gpu
    g = yahkv.f16_geometry(2, 1, 128, 16, 4)
    dev = yahkv.F16Pools(g)
    table = torch.tensor([[2, 1]], dtype=torch.int32, device="cuda")  # 32 positions
    x = np.arange(10 * 128, dtype=np.float32).reshape(1, 10, 1, 128) / 8.0
    yahkv.f16_append(dev, table, torch.tensor([28], dtype=torch.int32, device="cuda"), tensor(torch, x, "f32"),
                     tensor(torch, -x, "f32"))
    K, V = gather(yahkv, dev, [2, 1], 32)
    assert np.array_equal(K[28:31, 0], x[0, :3, 0].astype(np.float16))
    assert np.array_equal(K[31, 0], x[0, 9, 0].astype(np.float16))  # tokens 3..9 clamp to the last slot: 9 wins
    assert np.array_equal(V[31, 0], (-x[0, 9, 0]).astype(np.float16))


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("hd,pt", [(128, 16), (256, 32), (256, 64), (128, 64)])
def test_a_chunk_appended_at_once_equals_its_tokens_one_by_one(yahkv, torch_gpu, kind, hd, pt):
    """Chunks take the kernel that works run by run, single tokens the one that works element by element: the pools
    must come out the same, byte for byte, also where positions clamp at either end and where a chunk is padded."""
    torch = torch_gpu
    rng = np.random.default_rng(hd + pt)
    n_kv, stride, n_new = 2, 5, 70
    starts = [3, -4, stride * pt - 40, 17, pt]      # inside, before the start, past the end, odd, on a page edge
    valid = [70, 70, 70, 33, 9]
    B = len(starts)
    g = yahkv.f16_geometry(4, n_kv, hd, pt, B * stride)
    table = torch.from_numpy(rng.permutation(B * stride).astype(np.int32).reshape(B, stride)).cuda()
    k = rng.standard_normal((B, n_new, n_kv, hd)).astype(np.float32) * 3
    v = rng.standard_normal((B, n_new, n_kv, hd)).astype(np.float32) * 3
    tk, tv = tensor(torch, k, kind), tensor(torch, v, kind)
    at_once, one_by_one = yahkv.F16Pools(g, fill=0x5A), yahkv.F16Pools(g, fill=0x5A)
    yahkv.f16_append(at_once, table, torch.tensor(starts, dtype=torch.int32, device="cuda"), tk, tv,
                     n_valid=torch.tensor(valid, dtype=torch.int32, device="cuda"))
    for s in range(B):
        for i in range(valid[s]):
            yahkv.f16_append(one_by_one, table[s:s + 1], torch.tensor([starts[s] + i], dtype=torch.int32, device="cuda"),
                             tk[s:s + 1, i:i + 1].contiguous(), tv[s:s + 1, i:i + 1].contiguous())
    assert torch.equal(at_once.k, one_by_one.k)
    assert torch.equal(at_once.v, one_by_one.v)
    assert int((at_once.k != 0x5A).sum()) > 0


def closed_form(K, V, q, scale, n_q):
    """float64 softmax(q K^T scale) V over f16 K, V [n][H][D]; q [n_q][D]."""
    n_kv = K.shape[1]
    out = np.zeros((n_q, K.shape[2]))
    if K.shape[0] == 0:
        return out
    for h in range(n_q):
        kk, vv = K[:, h // (n_q // n_kv)].astype(np.float64), V[:, h // (n_q // n_kv)].astype(np.float64)
        sc = kk @ q[h].astype(np.float64) * scale
        p = np.exp(sc - sc.max())
        out[h] = (p / p.sum()) @ vv
    return out


CASES = [  # n_q, n_kv, hd, pt, lengths
    (8, 2, 128, 16, [513]),
    (24, 4, 256, 64, [1, 64, 65, 1000, 0, 4097]),
    (8, 1, 256, 32, [31, 33, 700]),
    (6, 2, 128, 64, [129, 2500]),
    (4, 4, 256, 16, [47, 900]),
    (16, 2, 128, 32, [3000, 17, 256]),
]


@pytest.mark.parametrize("n_q,n_kv,hd,pt,lens", CASES)
@pytest.mark.parametrize("qkind", ["bf16", "f32"])
def test_decode_against_the_closed_form(yahkv, torch_gpu, n_q, n_kv, hd, pt, lens, qkind):
    check_decode(yahkv, torch_gpu, n_q, n_kv, hd, pt, lens, qkind, n_q * 1000 + hd + pt)


@pytest.mark.parametrize("seed", range(12))
def test_decode_on_random_shapes_and_cuts(yahkv, torch_gpu, seed):
    """Random group sizes, head dims, page sizes, ragged and empty sequences, and the number of stretches a sequence
    is cut into forced from one per sequence to one per 128 keys: every cut gives the closed form."""
    rng = np.random.default_rng(1000 + seed)
    n_kv, group = int(rng.choice([1, 2, 4])), int(rng.integers(1, 9))
    hd, pt = int(rng.choice([128, 256])), int(rng.choice([16, 32, 64]))
    lens = [int(x) for x in rng.integers(0, 3000, int(rng.integers(1, 6)))]
    if max(lens) == 0:
        lens[0] = 1
    wgs = [0, 1, 64, 1000000][seed % 4]
    check_decode(yahkv, torch_gpu, n_kv * group, n_kv, hd, pt, lens, ["bf16", "f32", "f16"][seed % 3], seed,
                 opt=yahkv.decode_options(n_chunks=wgs) if wgs else None)


def check_decode(yahkv, torch, n_q, n_kv, hd, pt, lens, qkind, seed, opt=None):
    rng = np.random.default_rng(seed)
    B, max_len = len(lens), max(lens)
    pages = [(l + pt - 1) // pt for l in lens]
    stride = max(max(pages), 1)
    n_pages = sum(pages) + 2
    g = yahkv.f16_geometry(n_q, n_kv, hd, pt, n_pages)
    perm = rng.permutation(n_pages).astype(np.int32)
    table = np.full((B, stride), -7, np.int32)  # entries past a sequence's pages are never trusted
    o = 0
    for s, n in enumerate(pages):
        table[s, :n] = perm[o:o + n]
        o += n
    dev = yahkv.F16Pools(g, fill=0x7E)  # 0x7E7E is an f16 NaN: what lies past a sequence's end must not leak
    t_table = torch.from_numpy(table).cuda()
    src = [(rng.standard_normal((l, n_kv, hd)).astype(np.float32), rng.standard_normal((l, n_kv, hd)).astype(np.float32))
           for l in lens]
    for s, l in enumerate(lens):
        if l:
            yahkv.f16_append(dev, t_table[s:s + 1], torch.zeros(1, dtype=torch.int32, device="cuda"),
                             tensor(torch, src[s][0][None], "f32"), tensor(torch, src[s][1][None], "f32"))
    q = rng.standard_normal((B, n_q, hd)).astype(np.float32)
    if qkind == "bf16":
        q = to_bf16_f32(q)
    if qkind == "f16":
        q = q.astype(np.float16).astype(np.float32)
    gate = rng.standard_normal((B, n_q, hd)).astype(np.float32) if qkind == "f32" else None
    scale = 1.0 / np.sqrt(hd)
    out = yahkv.f16_decode_attend(dev, t_table, torch.tensor(lens, dtype=torch.int32, device="cuda"), max_len,
                                  tensor(torch, q, qkind), scale, opt=opt,
                                  gate=None if gate is None else torch.from_numpy(gate).cuda()).cpu().numpy()
    assert np.all(np.isfinite(out))
    for s, l in enumerate(lens):
        want = closed_form(src[s][0].astype(np.float16), src[s][1].astype(np.float16), q[s], scale, n_q)
        if gate is not None:
            want = want / (1.0 + np.exp(-gate[s].astype(np.float64)))
        if l == 0:
            assert np.all(out[s] == 0.0)
            continue
        err = np.abs(out[s] - want).max() / np.abs(want).max()
        assert err < 2e-3, (s, l, err)


def test_length_beyond_the_bound_is_clamped_and_arguments_are_checked(yahkv, torch_gpu):
    import ctypes as C
    torch = torch_gpu
    rng = np.random.default_rng(5)
    g = yahkv.f16_geometry(8, 2, 128, 16, 8)
    dev = yahkv.F16Pools(g)
    table = torch.from_numpy(rng.permutation(8).astype(np.int32)[None]).cuda()
    x = rng.standard_normal((1, 100, 2, 128)).astype(np.float32)
    yahkv.f16_append(dev, table, torch.zeros(1, dtype=torch.int32, device="cuda"), tensor(torch, x, "f32"),
                     tensor(torch, x, "f32"))
    q = tensor(torch, rng.standard_normal((1, 8, 128)).astype(np.float32), "f32")
    a = yahkv.f16_decode_attend(dev, table, torch.tensor([100], dtype=torch.int32, device="cuda"), 100, q, 0.1)
    b = yahkv.f16_decode_attend(dev, table, torch.tensor([100000], dtype=torch.int32, device="cuda"), 100, q, 0.1)
    assert torch.equal(a, b)
    g8 = yahkv.geometry(8, 8, 2, 128, 16, 8)  # a quantized geometry is not an f16 one
    assert yahkv.lib.yahkv_f16_pool_bytes(C.byref(g8)) == 0
    assert yahkv.lib.yahkv_f16_decode_workspace_bytes(C.byref(g8), 1, 100, None) == 0
    st = dev.struct()
    rc = yahkv.lib.yahkv_f16_decode_attend(C.byref(g), C.byref(st), table.data_ptr(), 8, None, 1, 100, q.data_ptr(), 0,
                                           0.1, None, a.data_ptr(), None, 0, None, None)
    assert rc == -1
    small = torch.empty(16, dtype=torch.uint8, device="cuda")
    rc = yahkv.lib.yahkv_f16_decode_attend(C.byref(g), C.byref(st), table.data_ptr(), 8, table.data_ptr(), 1, 100,
                                           q.data_ptr(), 0, 0.1, None, a.data_ptr(), small.data_ptr(), 16, None, None)
    assert rc == -4


@pytest.mark.parametrize("n_q,n_kv,hd,pt,prefix,chunk", [(24, 4, 256, 64, [700, 64, 0], 130), (8, 2, 128, 16, [33], 64),
                                                         (12, 4, 128, 32, [500, 1000], 70)])
def test_prefill_over_f16_pools(yahkv, torch_gpu, n_q, n_kv, hd, pt, prefix, chunk):
    """Causal attention of a chunk over prefix + chunk in f16 pools, against the float64 closed form over the f16
    values: the pools' values reach the matrix unit as they are, the numerators are f16; bound 2e-3."""
    torch = torch_gpu
    rng = np.random.default_rng(hd + pt + chunk)
    B = len(prefix)
    pages = [(p + chunk + pt - 1) // pt for p in prefix]
    n_pages = sum(pages)
    g = yahkv.f16_geometry(n_q, n_kv, hd, pt, n_pages)
    perm = rng.permutation(n_pages).astype(np.int32)
    table = np.zeros((B, max(pages)), np.int32)
    o = 0
    for s, n in enumerate(pages):
        table[s, :n] = perm[o:o + n]
        o += n
    dev = yahkv.F16Pools(g, fill=0x7E)
    t_table = torch.from_numpy(table).cuda()
    src = [(rng.standard_normal((p + chunk, n_kv, hd)).astype(np.float32), rng.standard_normal((p + chunk, n_kv, hd)).astype(np.float32))
           for p in prefix]
    for s in range(B):
        yahkv.f16_append(dev, t_table[s:s + 1], torch.zeros(1, dtype=torch.int32, device="cuda"),
                         tensor(torch, src[s][0][None], "f32"), tensor(torch, src[s][1][None], "f32"))
    q = to_bf16_f32(rng.standard_normal((B, chunk, n_q, hd)).astype(np.float32))
    scale = 1.0 / np.sqrt(hd)
    out = yahkv.f16_prefill_attend(dev, t_table, torch.tensor(prefix, dtype=torch.int32, device="cuda"), max(prefix),
                                   tensor(torch, q, "bf16"), scale).float().cpu().numpy()
    assert np.all(np.isfinite(out))
    worst = 0.0
    for s in range(B):
        K, V = src[s][0].astype(np.float16), src[s][1].astype(np.float16)
        for t in (0, chunk // 2, chunk - 1):
            n = prefix[s] + t + 1
            want = closed_form(K[:n], V[:n], q[s, t], scale, n_q)
            worst = max(worst, float(np.abs(out[s, t] - want).max() / np.abs(want).max()))
    assert worst < 2e-3, worst


def test_prefill_over_f16_pools_checks_its_arguments(yahkv, torch_gpu):
    import ctypes as C
    torch = torch_gpu
    g = yahkv.f16_geometry(8, 2, 128, 16, 8)
    dev = yahkv.F16Pools(g)
    table = torch.arange(8, dtype=torch.int32, device="cuda")[None]
    prefix = torch.zeros(1, dtype=torch.int32, device="cuda")
    q = torch.zeros((1, 32, 8, 128), dtype=torch.bfloat16, device="cuda")
    out = torch.empty_like(q)
    need = yahkv.lib.yahkv_f16_prefill_workspace_bytes(C.byref(g), 1, 0, 32)
    assert need > 0
    g8 = yahkv.geometry(8, 8, 2, 128, 16, 8)
    assert yahkv.lib.yahkv_f16_prefill_workspace_bytes(C.byref(g8), 1, 0, 32) == 0
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    st = dev.struct()

    def call(geom, workspace, n_bytes, chunk=32):
        return yahkv.lib.yahkv_f16_prefill_attend(C.byref(geom), C.byref(st), table.data_ptr(), 8, prefix.data_ptr(), 1,
                                                  0, chunk, q.data_ptr(), 0.1, None, out.data_ptr(), 2,
                                                  workspace, n_bytes, None)
    assert call(g8, ws.data_ptr(), need) == -2           # a quantized geometry
    assert call(g, None, 0) == -1                        # the workspace is required
    assert call(g, ws.data_ptr(), need - 1) == -4        # and must hold the tile images
    assert call(g, ws.data_ptr(), need, chunk=16 * 8 + 1) == -1   # more chunk positions than the table has rows for
    assert call(g, ws.data_ptr(), need) == 0
    torch.cuda.synchronize()
