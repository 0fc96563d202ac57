"""GPU append against the CPU oracle: pool bytes, scales and untouched bytes bit-exact, through the C ABI."""
import numpy as np
import pytest

import oracle
from helpers import bf16_bits, make_tables, to_bf16_f32, to_f16_f32

pytestmark = pytest.mark.gpu


def torch_src(torch, x, kind):
    """x f32 numpy, already representable in `kind` -> cuda tensor of that dtype."""
    if kind == "f32":
        return torch.from_numpy(np.ascontiguousarray(x, np.float32)).cuda()
    if kind == "f16":
        return torch.from_numpy(x.astype(np.float16)).cuda()
    return torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)


def same_pools(dev, host):
    got = dev.numpy()
    for name, want in host.arrays().items():
        assert np.array_equal(got[name], want), f"pool {name} differs in {(got[name] != want).sum()} elements"


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt,kind", [
    (8, 8, 2, 128, 16, "f16"), (8, 24, 4, 256, 64, "bf16"), (8, 24, 4, 256, 64, "f32"),
    (4, 24, 4, 256, 64, "bf16"), (4, 8, 2, 128, 16, "f16"), (8, 6, 1, 128, 32, "f32")])
def test_chunk_then_token_append_bit_exact(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt, kind):
    torch = torch_gpu
    rng = np.random.default_rng(100 + fmt + hd + pt)
    lens = [3 * pt + 5, pt - 1, 2 * pt]
    chunk = max(lens)
    pages = [(n + 1 + pt - 1) // pt for n in lens]
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, sum(pages) + 3)
    table = make_tables(rng, pages, g.n_pages)
    rnd = {"f32": lambda x: x.astype(np.float32), "f16": to_f16_f32, "bf16": to_bf16_f32}[kind]
    K = rnd(rng.standard_normal((3, chunk + 1, n_kv, hd)) * 10.0 ** rng.uniform(-2, 2, (3, chunk + 1, n_kv, 1)))
    V = rnd(rng.standard_normal((3, chunk + 1, n_kv, hd)))
    host = oracle.HostPools(g, fill=0xA5)
    dev = yahkv.DevicePools(yahkv.geometry(fmt, n_q, n_kv, hd, pt, g.n_pages), fill=0xA5)
    t_table = torch.from_numpy(table).cuda()
    zeros = torch.zeros(3, dtype=torch.int32, device="cuda")
    nv = torch.tensor(lens, dtype=torch.int32, device="cuda")
    # a padded chunk (n_valid rows real), then one token per sequence at its own position
    oracle.append(host, table, [0, 0, 0], lens, K[:, :chunk], V[:, :chunk])
    yahkv.append(dev, t_table, zeros, torch_src(torch, K[:, :chunk], kind), torch_src(torch, V[:, :chunk], kind), n_valid=nv)
    same_pools(dev, host)
    knew = np.stack([K[s, lens[s]] for s in range(3)])[:, None]
    vnew = np.stack([V[s, lens[s]] for s in range(3)])[:, None]
    oracle.append(host, table, lens, None, knew, vnew)
    yahkv.append(dev, t_table, nv, torch_src(torch, knew, kind), torch_src(torch, vnew, kind))
    same_pools(dev, host)
    # ggml block order through the library's gather == contiguous quantize of the same rows
    quant = oracle.quantize_q8_0 if fmt == 8 else oracle.quantize_q4_0
    for s in range(3):
        k, v = yahkv.gather_blocks(dev, t_table[s], lens[s] + 1)
        bb = 34 if fmt == 8 else 18
        assert np.array_equal(k.cpu().numpy().reshape(-1, bb), quant(K[s, :lens[s] + 1]))
        assert np.array_equal(v.cpu().numpy().reshape(-1, bb), quant(V[s, :lens[s] + 1]))


def test_q8_0_golden_blocks_from_the_reference(yahkv, torch_gpu, golden):
    """The reference's own QuantizeQ8_0 outputs (edge blocks included) reproduced by the GPU append, f32 source."""
    torch = torch_gpu
    x, want = golden["q8_in"], golden["q8_out"]
    n_kv, hd, pt = 2, 128, 16
    per_tok = n_kv * hd // 32
    n_tok = (len(x) + per_tok - 1) // per_tok
    xp = np.zeros((n_tok * per_tok, 32), np.float32)
    xp[:len(x)] = x
    src = xp.reshape(1, n_tok, n_kv, hd)
    pages = (n_tok + pt - 1) // pt
    g = yahkv.geometry(8, 8, n_kv, hd, pt, pages)
    dev = yahkv.DevicePools(g)
    table = torch.from_numpy(np.random.default_rng(0).permutation(pages).astype(np.int32)[None]).cuda()
    t = torch.from_numpy(src).cuda()
    yahkv.append(dev, table, torch.zeros(1, dtype=torch.int32, device="cuda"), t, t)
    k, v = yahkv.gather_blocks(dev, table[0], n_tok)
    assert np.array_equal(k.cpu().numpy().reshape(-1, 34)[:len(x)], want)
    assert np.array_equal(v.cpu().numpy().reshape(-1, 34)[:len(x)], want)


@pytest.mark.parametrize("kind", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("hd,pt,n_new", [(128, 16, 1), (256, 64, 1), (256, 64, 64), (128, 32, 24)])
def test_q4_0_known_answers_through_the_append(yahkv, torch_gpu, kind, hd, pt, n_new):
    """The hand-computed q4_0 blocks of tests/q4_known_answers.py (ties, clip, first of two equal magnitudes at every
    pair of positions) through yahkv_append, token by token and as chunks, K and V, then read back as ggml blocks."""
    torch = torch_gpu
    from q4_known_answers import known_answers
    x, want, names = known_answers()
    n_kv = 2
    per_tok = n_kv * hd // 32
    n_tok = (len(x) + per_tok - 1) // per_tok
    n_tok = (n_tok + n_new - 1) // n_new * n_new
    xp = np.zeros((n_tok * per_tok, 32), np.float32)
    xp[:len(x)] = x
    src = xp.reshape(1, n_tok, n_kv, hd)
    pages = (n_tok + pt - 1) // pt
    g = yahkv.geometry(4, 2 * n_kv, n_kv, hd, pt, pages)
    dev = yahkv.DevicePools(g, fill=0x5A)
    table = torch.from_numpy(np.random.default_rng(1).permutation(pages).astype(np.int32)[None]).cuda()
    t = torch_src(torch, src, kind)
    for o in range(0, n_tok, n_new):
        yahkv.append(dev, table, torch.tensor([o], dtype=torch.int32, device="cuda"), t[:, o:o + n_new], t[:, o:o + n_new])
    k, v = yahkv.gather_blocks(dev, table[0], n_tok)
    for what, got in (("K", k), ("V", v)):
        got = got.cpu().numpy().reshape(-1, 18)[:len(x)]
        for i in np.flatnonzero((got != want).any(1)):
            raise AssertionError(f"{what} block '{names[i]}': got {got[i].tolist()}, want {want[i].tolist()}")


def test_append_clamps_bad_positions_and_pages(yahkv, torch_gpu):
    """Positions past the table and page ids outside the pool are clamped, never written out of bounds."""
    torch = torch_gpu
    g = yahkv.geometry(8, 8, 2, 128, 16, 4)
    dev = yahkv.DevicePools(g, fill=0x11)
    guard = {n: getattr(dev, n).clone() for n in ("kq", "ks", "vq", "vs")}
    table = torch.tensor([[99, -5]], dtype=torch.int32, device="cuda")
    src = torch.randn(1, 1, 2, 128, device="cuda")
    for pos in (10 ** 6, -7):
        yahkv.append(dev, table, torch.tensor([pos], dtype=torch.int32, device="cuda"), src, src)
    torch.cuda.synchronize()
    changed = sum(int((getattr(dev, n) != guard[n]).sum()) for n in guard)
    assert 0 < changed <= 2 * 2 * (2 * 128 + 2 * 4 * 2)   # two slots at most, inside the pools


def test_append_rejects_bad_arguments(yahkv, torch_gpu):
    torch = torch_gpu
    with pytest.raises(yahkv.YahkvError):
        yahkv.geometry(8, 24, 4, 192, 64, 8)            # no kernel for head_dim 192
    with pytest.raises(yahkv.YahkvError):
        yahkv.geometry(8, 24, 5, 256, 64, 8)            # 24 query heads over 5 kv heads
    g = yahkv.geometry(8, 8, 2, 128, 16, 4)
    dev = yahkv.DevicePools(g)
    st = dev.struct()
    import ctypes as C
    rc = yahkv.lib.yahkv_append(C.byref(g), C.byref(st), None, 1, None, None, 1, 1, None, None, 0, None)
    assert rc == -1


@pytest.mark.parametrize("fmt,pt,n_new", [(8, 64, 40), (4, 16, 40), (8, 32, 40), (8, 64, 6), (4, 32, 7)])
def test_chunk_positions_clamp_like_a_loop_over_the_tokens(yahkv, torch_gpu, fmt, pt, n_new):
    """A chunk that runs past the table's last position, and one that starts before position 0: every token goes to
    its clamped position, and where several clamp to the same slot the last one stays, as in the oracle's loop (chunks
    of 40 tokens go page by page, those of 6 or 7 token by token)."""
    torch = torch_gpu
    rng = np.random.default_rng(fmt + pt + n_new)
    n_kv, hd, stride = 2, 128, 3
    g = oracle.geometry(fmt, n_kv, n_kv, hd, pt, 3 * stride + 1)
    table = make_tables(rng, [stride] * 3, g.n_pages)
    host = oracle.HostPools(g, fill=0x3C)
    dev = yahkv.DevicePools(yahkv.geometry(fmt, n_kv, n_kv, hd, pt, g.n_pages), fill=0x3C)
    over = 25 if n_new == 40 else 3
    start = np.array([stride * pt - over, -7 if n_new == 40 else -3, stride * pt + 100], np.int32)    # over the end, before 0, all past the end
    valid = np.array([n_new, 33, 12] if n_new == 40 else [n_new, n_new - 1, 4], np.int32)
    K = to_bf16_f32(rng.standard_normal((3, n_new, n_kv, hd)))
    V = to_bf16_f32(rng.standard_normal((3, n_new, n_kv, hd)))
    oracle.append(host, table, start, valid, K, V)
    yahkv.append(dev, torch.from_numpy(table).cuda(), torch.from_numpy(start).cuda(), torch_src(torch, K, "bf16"),
                 torch_src(torch, V, "bf16"), n_valid=torch.from_numpy(valid).cuda())
    same_pools(dev, host)
