"""The benchmark configurations that the other GPU tests do not reach at their own geometry and size, through the
C ABI, in the manner of the reference's checker (engine/gpu/loom/tools/dattn_q_check.py:140-256: seeded inputs, a
scrambled page table, pools filled with poison first, appended bytes bit-exact, attention against the float64
closed form over the dequantized blocks):
  config 2   one sequence of 32768 tokens, q8_0, 24 Q / 4 KV heads, head_dim 256, 64-token pages, a 1024-page pool
             of which a seeded permutation hands out 512 (+ 1 for the appended token), bf16 query
  config 3   the headline: 64 sequences with lengths uniform in [1024, 65536], q8_0, one shared pool sized to fit exactly
             through the page allocator and shuffled; the source rows of the shortest, the median, the longest sequence
             and of one whose length is a multiple of 64 (its step's token opens a new page) are kept and their pool
             blocks held to the oracle's quantizer bit for bit; then one decode step (append + attention), those
             sequences against the closed form, and the new token not visible one step earlier
  config 5   q4_0, batch 16, the same heads, K with 8 seeded outlier channels per head scaled x 20; at 2048 tokens per
             sequence against the oracle, and at the full 131072 tokens per sequence against the closed form on the
             gathered blocks of two sequences; one token appended per sequence before the attention
  config 4   chunked prefill, q8_0, 8 sequences with 16384 tokens of prefix and a chunk of 2048 each, at full size:
             sampled (position, head) rows of three sequences against the closed form in exact arithmetic
"""
import numpy as np
import pytest

import oracle
from helpers import bf16_bits, closed_form, make_tables, rel_err, to_bf16_f32

pytestmark = pytest.mark.gpu
TOL = 2e-3
NQ, NKV, HD, PT = 24, 4, 256, 64


def bf16_cuda(torch, x):
    return torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)


def closed_from_blocks(yahkv, dev, t_row, n, q, scale, fmt):
    """Float64 closed form over what the library's own pools hold for one sequence (its blocks in ggml order)."""
    k, v = yahkv.gather_blocks(dev, t_row, n)
    bb = 34 if fmt == 8 else 18
    deq = oracle.dequantize_q8_0 if fmt == 8 else oracle.dequantize_q4_0
    Kd = deq(k.cpu().numpy().reshape(-1, bb)).reshape(n, NKV, HD)
    Vd = deq(v.cpu().numpy().reshape(-1, bb)).reshape(n, NKV, HD)
    return closed_form(Kd, Vd, q, scale)


def test_config2_one_sequence_of_32768_tokens(yahkv, torch_gpu):
    torch = torch_gpu
    rng = np.random.default_rng(22)
    n, pool_pages = 32768, 1024
    g = oracle.geometry(8, NQ, NKV, HD, PT, pool_pages)
    table = rng.permutation(pool_pages).astype(np.int32)[None, :n // PT + 1]        # 513 of the 1024 pages
    K = to_bf16_f32(rng.standard_normal((1, n + 1, NKV, HD)))
    V = to_bf16_f32(rng.standard_normal((1, n + 1, NKV, HD)))
    q = to_bf16_f32(rng.standard_normal((1, NQ, HD)))
    host = oracle.HostPools(g, fill=0x7F)                                           # f16 0x7F7F is NaN: poison
    oracle.append(host, table, [0], None, K, V)
    dev = yahkv.DevicePools(yahkv.geometry(8, NQ, NKV, HD, PT, pool_pages), fill=0x7F)
    t_table = torch.from_numpy(table).cuda()
    for o in range(0, n, 8192):                                                     # the prefix in chunks ...
        yahkv.append(dev, t_table, torch.tensor([o], dtype=torch.int32, device="cuda"),
                     bf16_cuda(torch, K[:, o:o + 8192]), bf16_cuda(torch, V[:, o:o + 8192]))
    yahkv.append(dev, t_table, torch.tensor([n], dtype=torch.int32, device="cuda"),  # ... and the step's token
                 bf16_cuda(torch, K[:, n:]), bf16_cuda(torch, V[:, n:]))
    got_pools = dev.numpy()
    for name, want in host.arrays().items():
        assert np.array_equal(got_pools[name], want), f"pool {name}: written bytes or untouched poison differ"
    scale = 1.0 / 16
    lens = torch.tensor([n + 1], dtype=torch.int32, device="cuda")
    out = yahkv.decode_attend(dev, t_table, lens, n + 1, bf16_cuda(torch, q), scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got))
    want = closed_from_blocks(yahkv, dev, t_table[0], n + 1, q[0], scale, 8)
    err = rel_err(got[0], want)
    assert err < TOL, err
    assert rel_err(got, oracle.decode_attend(host, table, [n + 1], q, scale)) < TOL
    # the appended token counts from its own step on, not before
    prev = yahkv.decode_attend(dev, t_table, lens - 1, n + 1, bf16_cuda(torch, q), scale).cpu().numpy()
    assert rel_err(prev[0], closed_from_blocks(yahkv, dev, t_table[0], n, q[0], scale, 8)) < TOL
    assert np.abs(prev - got).max() > 0


def test_config3_ragged_batch_of_64_at_full_size(yahkv, torch_gpu):
    torch = torch_gpu
    rng = np.random.default_rng(4)
    B = 64
    lens = rng.integers(1024, 65537, B).astype(np.int32)
    order = np.argsort(lens)
    crossing = int(order[B // 3])
    lens[crossing] = (int(lens[crossing]) // PT) * PT          # the step's token is this sequence's first on a new page
    order = np.argsort(lens)
    kept = sorted({int(order[0]), int(order[B // 2]), int(order[-1]), crossing})
    pages = (lens + 1 + PT - 1) // PT
    n_pages = int(pages.sum())                                 # the pool fits the job exactly
    g = yahkv.geometry(8, NQ, NKV, HD, PT, n_pages)
    alloc = yahkv.PagePool(n_pages)
    alloc.shuffle(4)
    table = np.zeros((B, int(pages.max())), np.int32)
    for s_, n_ in enumerate(pages):
        table[s_, :n_] = alloc.alloc(int(n_))
    assert alloc.free_count == 0
    yahkv.validate_page_table(g, table, lens + 1)
    dev = yahkv.DevicePools(g, fill=0x7F)
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(4)
    src = {}
    for s_ in range(B):
        ks, vs = [], []
        for o in range(0, int(lens[s_]), 8192):
            n_ = min(8192, int(lens[s_]) - o)
            k = torch.randn((1, n_, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            v = torch.randn((1, n_, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            yahkv.append(dev, t_table[s_:s_ + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
            if s_ in kept:
                ks.append(k[0].float().cpu().numpy()), vs.append(v[0].float().cpu().numpy())
        if s_ in kept:
            src[s_] = (np.concatenate(ks), np.concatenate(vs))
    knew = to_bf16_f32(rng.standard_normal((B, NKV, HD)))
    vnew = to_bf16_f32(rng.standard_normal((B, NKV, HD)))
    q = to_bf16_f32(rng.standard_normal((B, NQ, HD)))
    scale = 1.0 / 16
    t_lens = torch.from_numpy(lens).cuda()
    max_len = int(lens.max()) + 1
    opt = yahkv.decode_options()
    ws = torch.empty(yahkv.decode_workspace_bytes(g, B, max_len, opt), dtype=torch.uint8, device="cuda")
    yahkv.decode_calibrate(dev, t_table, t_lens, max_len, bf16_cuda(torch, q), ws, opt, rounds=2)   # unequal XCD shares, as the bench runs
    before = yahkv.decode_attend(dev, t_table, t_lens, max_len, bf16_cuda(torch, q), scale, workspace=ws, opt=opt).cpu().numpy()
    out = yahkv.decode_step(dev, t_table, t_lens + 1, max_len, bf16_cuda(torch, knew), bf16_cuda(torch, vnew),
                            bf16_cuda(torch, q), scale, workspace=ws, opt=opt)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got))
    for s_ in kept:
        n_ = int(lens[s_])
        k, v = yahkv.gather_blocks(dev, t_table[s_], n_ + 1)
        kb, vb = k.cpu().numpy(), v.cpu().numpy()
        # pool bytes of the whole sequence against the oracle's quantizer on the kept source rows, and the step's token
        assert np.array_equal(kb[:n_].reshape(-1, 34), oracle.quantize_q8_0(src[s_][0])), f"sequence {s_}: K blocks"
        assert np.array_equal(vb[:n_].reshape(-1, 34), oracle.quantize_q8_0(src[s_][1])), f"sequence {s_}: V blocks"
        assert np.array_equal(kb[n_].reshape(-1, 34), oracle.quantize_q8_0(knew[s_])), f"sequence {s_}: the step's K"
        assert np.array_equal(vb[n_].reshape(-1, 34), oracle.quantize_q8_0(vnew[s_])), f"sequence {s_}: the step's V"
        Kd = oracle.dequantize_q8_0(kb.reshape(-1, 34)).reshape(n_ + 1, NKV, HD)
        Vd = oracle.dequantize_q8_0(vb.reshape(-1, 34)).reshape(n_ + 1, NKV, HD)
        err = rel_err(got[s_], closed_form(Kd, Vd, q[s_], scale))
        assert err < TOL, (s_, n_, err)
        assert rel_err(before[s_], closed_form(Kd[:n_], Vd[:n_], q[s_], scale)) < TOL, (s_, "one step earlier")
        assert np.abs(before[s_] - got[s_]).max() > 0
    assert int(lens[crossing]) % PT == 0 and pages[crossing] == int(lens[crossing]) // PT + 1   # the token's own page
    # every other row of the batch: the step's attention against the closed form over that sequence's own blocks
    worst = 0.0
    for s_ in range(B):
        if s_ in kept:
            continue
        n_ = int(lens[s_]) + 1
        k, v = yahkv.gather_blocks(dev, t_table[s_], n_)
        Kd = oracle.dequantize_q8_0(k.cpu().numpy().reshape(-1, 34)).reshape(n_, NKV, HD)
        Vd = oracle.dequantize_q8_0(v.cpu().numpy().reshape(-1, 34)).reshape(n_, NKV, HD)
        worst = max(worst, rel_err(got[s_], closed_form(Kd, Vd, q[s_], scale)))
    print(f"config 3, the other {B - len(kept)} rows against the closed form: {worst:.2e}")
    assert worst < TOL


def outlier_scales(rng):
    s = np.ones((NKV, HD), np.float32)
    for h in range(NKV):
        s[h, rng.permutation(HD)[:8]] = 20.0
    return s


def test_config5_q4_0_outlier_channels_against_the_oracle(yahkv, torch_gpu):
    """16 sequences of 2048 tokens (+ 1 appended): pools bit-exact, attention within tolerance of the oracle."""
    torch = torch_gpu
    rng = np.random.default_rng(55)
    B, n = 16, 2048
    pages = [(n + 1 + PT - 1) // PT] * B
    g = oracle.geometry(4, NQ, NKV, HD, PT, sum(pages))
    table = make_tables(rng, pages, g.n_pages)
    outl = outlier_scales(rng)
    K = to_bf16_f32(rng.standard_normal((B, n + 1, NKV, HD)).astype(np.float32) * outl)
    V = to_bf16_f32(rng.standard_normal((B, n + 1, NKV, HD)))
    q = to_bf16_f32(rng.standard_normal((B, NQ, HD)))
    host = oracle.HostPools(g, fill=0x7F)
    oracle.append(host, table, [0] * B, None, K, V)
    dev = yahkv.DevicePools(yahkv.geometry(4, NQ, NKV, HD, PT, g.n_pages), fill=0x7F)
    t_table = torch.from_numpy(table).cuda()
    zeros = torch.zeros(B, dtype=torch.int32, device="cuda")
    yahkv.append(dev, t_table, zeros, bf16_cuda(torch, K[:, :n]), bf16_cuda(torch, V[:, :n]))
    yahkv.append(dev, t_table, zeros + n, bf16_cuda(torch, K[:, n:]), bf16_cuda(torch, V[:, n:]))
    got_pools = dev.numpy()
    for name, want in host.arrays().items():
        assert np.array_equal(got_pools[name], want), f"pool {name} differs"
    # the outlier channels did what they are there for: their blocks' scales are large, their block-mates coarse
    kblocks, _ = oracle.gather_blocks(host, table[0], 64)
    d = np.abs(kblocks[..., :2].copy().view(np.float16).astype(np.float32))[..., 0]      # [tok][H][NB]
    hot = np.zeros((NKV, HD // 32), bool)
    for h in range(NKV):
        hot[h, np.flatnonzero(outl[h] > 1) // 32] = True
    assert d[:, hot].mean() > 4 * d[:, ~hot].mean()
    scale = 1.0 / 16
    out = yahkv.decode_attend(dev, t_table, zeros + n + 1, n + 1, bf16_cuda(torch, q), scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got))
    want = oracle.decode_attend(host, table, [n + 1] * B, q, scale)
    for s in range(B):
        assert rel_err(got[s], want[s]) < TOL, s


def test_config5_q4_0_batch16_of_131072_tokens(yahkv, torch_gpu):
    """The full size: 16 x 131072 tokens, the pool sized to fit exactly, one global shuffle of the pages; the K / V
    source is drawn on the GPU (torch supplies the random numbers) and quantized by the library's own append, which the
    test above and the append tests hold to the oracle bit for bit. Checked: the closed form over the gathered blocks
    of two sequences, and the blocks of every sequence's appended token against the oracle's quantizer."""
    torch = torch_gpu
    rng = np.random.default_rng(56)
    B, n = 16, 131072
    per_seq = (n + 1 + PT - 1) // PT
    n_pages = B * per_seq
    g = yahkv.geometry(4, NQ, NKV, HD, PT, n_pages)
    table = make_tables(rng, [per_seq] * B, n_pages)
    yahkv.validate_page_table(g, table, np.full(B, n + 1, np.int32))
    dev = yahkv.DevicePools(g, fill=0x7F)
    t_table = torch.from_numpy(table).cuda()
    outl = torch.from_numpy(outlier_scales(rng)).cuda()
    gen = torch.Generator(device="cuda").manual_seed(56)
    for s in range(B):
        for o in range(0, n, 16384):
            k = (torch.randn((1, 16384, NKV, HD), generator=gen, device="cuda") * outl).to(torch.bfloat16)
            v = torch.randn((1, 16384, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            yahkv.append(dev, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
    knew = to_bf16_f32(rng.standard_normal((B, 1, NKV, HD)).astype(np.float32) * outl.cpu().numpy())
    vnew = to_bf16_f32(rng.standard_normal((B, 1, NKV, HD)))
    lens = torch.full((B,), n, dtype=torch.int32, device="cuda")
    yahkv.append(dev, t_table, lens, bf16_cuda(torch, knew), bf16_cuda(torch, vnew))
    q = to_bf16_f32(rng.standard_normal((B, NQ, HD)))
    scale = 1.0 / 16
    out = yahkv.decode_attend(dev, t_table, lens + 1, n + 1, bf16_cuda(torch, q), scale)
    torch.cuda.synchronize()
    got = out.cpu().numpy()
    assert np.all(np.isfinite(got))
    for s in range(B):                                        # the step's token, bit for bit
        k, v = yahkv.gather_blocks(dev, t_table[s], n + 1)
        assert np.array_equal(k[n].cpu().numpy().reshape(-1, 18), oracle.quantize_q4_0(knew[s, 0])), s
        assert np.array_equal(v[n].cpu().numpy().reshape(-1, 18), oracle.quantize_q4_0(vnew[s, 0])), s
        del k, v
    for s in (0, B - 1):
        want = closed_from_blocks(yahkv, dev, t_table[s], n + 1, q[s], scale, 4)
        err = rel_err(got[s], want)
        assert err < TOL, (s, err)


def test_config4_prefill_chunk_of_2048_on_16384_tokens_of_prefix(yahkv, torch_gpu):
    """8 x (16384 + 2048), q8_0: the K / V source is drawn on the GPU and quantized by the library's own append (held
    to the oracle bit for bit elsewhere); the chunk goes through append, tile decode and attention as one prefill
    step does. Rows are checked against float64 arithmetic on the dequantized blocks, nothing of the f16 operands
    modelled: measured 6.3e-4, the bar is the path's 2e-3."""
    torch = torch_gpu
    rng = np.random.default_rng(44)
    B, prefix, chunk = 8, 16384, 2048
    n = prefix + chunk
    per_seq = n // PT
    g = yahkv.geometry(8, NQ, NKV, HD, PT, B * per_seq)
    table = make_tables(rng, [per_seq] * B, B * per_seq)
    dev = yahkv.DevicePools(g, fill=0x7F)
    t_table = torch.from_numpy(table).cuda()
    gen = torch.Generator(device="cuda").manual_seed(44)
    for s in range(B):
        for o in range(0, prefix, 8192):
            k = torch.randn((1, 8192, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            v = torch.randn((1, 8192, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
            yahkv.append(dev, t_table[s:s + 1], torch.tensor([o], dtype=torch.int32, device="cuda"), k, v)
    t_prefix = torch.full((B,), prefix, dtype=torch.int32, device="cuda")
    knew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    vnew = torch.randn((B, chunk, NKV, HD), generator=gen, device="cuda").to(torch.bfloat16)
    q = torch.randn((B, chunk, NQ, HD), generator=gen, device="cuda").to(torch.bfloat16)
    scale = 1.0 / 16
    yahkv.append(dev, t_table, t_prefix, knew, vnew)
    out = yahkv.prefill_attend(dev, t_table, t_prefix, prefix, q, scale, out_dtype=torch.float16)
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out).all())
    worst = 0.0
    for s in (0, 3, B - 1):
        k, v = yahkv.gather_blocks(dev, t_table[s], n)
        Kd = oracle.dequantize_q8_0(k.cpu().numpy().reshape(-1, 34)).reshape(n, NKV, HD).astype(np.float64)
        Vd = oracle.dequantize_q8_0(v.cpu().numpy().reshape(-1, 34)).reshape(n, NKV, HD).astype(np.float64)
        for t in (0, 1, 63, 64, chunk // 3, chunk // 2, chunk - 65, chunk - 1):
            for h in (0, 7, 13, NQ - 1):
                kv = h // (NQ // NKV)
                sc = Kd[:prefix + t + 1, kv] @ q[s, t, h].double().cpu().numpy() * scale
                p = np.exp(sc - sc.max())
                want = (p / p.sum()) @ Vd[:prefix + t + 1, kv]
                got = out[s, t, h].float().cpu().numpy()
                worst = max(worst, float(np.abs(got - want).max() / np.abs(want).max()))
    assert worst < TOL, worst
