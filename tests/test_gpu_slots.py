"""Shared prefixes and slots on the paged pools: a forked sequence shares the prefix's full pages (owner counts) and
gets a private copy of the partly filled last page; a slot (the pages of one sequence, packed) loads into other
physical pages. Checks are byte-for-byte on the gathered blocks; attention outputs agree within the decode kernel's
run-to-run variation."""
import numpy as np
import pytest

import oracle
from helpers import bf16_bits, rel_err, to_bf16_f32

pytestmark = pytest.mark.gpu


def fill(yahkv, torch, fmt, n_q, n_kv, hd, pt, n, n_pages, seed):
    rng = np.random.default_rng(seed)
    g = yahkv.geometry(fmt, n_q, n_kv, hd, pt, n_pages)
    dev = yahkv.DevicePools(g, fill=0x33)
    alloc = yahkv.PagePool(n_pages)
    alloc.shuffle(seed)
    pages = alloc.alloc((n + pt - 1) // pt)
    k = to_bf16_f32(rng.standard_normal((1, n, n_kv, hd)))
    v = to_bf16_f32(rng.standard_normal((1, n, n_kv, hd)))
    to_t = lambda x: torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)
    row = torch.tensor([pages], dtype=torch.int32, device="cuda")
    yahkv.append(dev, row, torch.zeros(1, dtype=torch.int32, device="cuda"), to_t(k), to_t(v))
    return g, dev, alloc, pages, rng, to_t


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt", [(8, 24, 4, 256, 64), (4, 8, 2, 128, 16)])
def test_fork_shares_full_pages_and_copies_the_last(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt):
    torch = torch_gpu
    n = 3 * pt + 5                                        # three full pages and a partly filled one
    g, dev, alloc, pages, rng, to_t = fill(yahkv, torch, fmt, n_q, n_kv, hd, pt, n, 12, seed=fmt + hd)
    # fork: share the full pages, copy the last
    child_last = alloc.alloc(1)
    alloc.retain(pages[:3])
    yahkv.copy_pages(dev, torch.tensor(pages[3:], dtype=torch.int32, device="cuda"),
                     torch.tensor(child_last, dtype=torch.int32, device="cuda"))
    child = pages[:3] + child_last
    assert [alloc.refcount(p) for p in child] == [2, 2, 2, 1]
    rows = torch.tensor([pages, child], dtype=torch.int32, device="cuda")
    # both continue with different tokens
    k2 = to_bf16_f32(rng.standard_normal((2, 4, n_kv, hd)))
    v2 = to_bf16_f32(rng.standard_normal((2, 4, n_kv, hd)))
    yahkv.append(dev, rows, torch.full((2,), n, dtype=torch.int32, device="cuda"), to_t(k2), to_t(v2))
    kp, vp = yahkv.gather_blocks(dev, rows[0], n + 4)
    kc, vc = yahkv.gather_blocks(dev, rows[1], n + 4)
    assert torch.equal(kp[:n], kc[:n]) and torch.equal(vp[:n], vc[:n])          # the shared prefix
    assert not torch.equal(kp[n:], kc[n:])                                       # their own continuations
    # the child's continuation equals quantizing its tokens alone
    bb = 34 if fmt == 8 else 18
    quant = oracle.quantize_q8_0 if fmt == 8 else oracle.quantize_q4_0
    want = quant(k2[1].reshape(-1, 32)).reshape(4, n_kv, hd // 32, bb)
    assert np.array_equal(kc[n:].cpu().numpy(), want)
    # the parent ends: shared pages stay with the child
    alloc.free(pages)
    assert [alloc.refcount(p) for p in child] == [1, 1, 1, 1] and alloc.refcount(pages[3]) == 0


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt", [(8, 24, 4, 256, 64), (4, 8, 2, 128, 32)])
def test_slot_round_trip_into_other_pages(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt):
    torch = torch_gpu
    n = 5 * pt - 7
    g, dev, alloc, pages, rng, to_t = fill(yahkv, torch, fmt, n_q, n_kv, hd, pt, n, 16, seed=fmt * 3 + pt)
    row = torch.tensor(pages, dtype=torch.int32, device="cuda")
    slot = yahkv.slot_pack(dev, row, len(pages), n)
    host = slot.cpu().numpy()                              # what a file would hold
    assert yahkv.slot_check(g, host) == (len(pages), n)
    assert host[:8].tobytes() == b"YKVSLOT1"
    with pytest.raises(yahkv.YahkvError) as e:             # another geometry refuses the slot
        yahkv.slot_check(yahkv.geometry(fmt, n_q, n_kv, hd, 16 if pt != 16 else 32, 16), host)
    assert e.value.status == -2
    bad = host.copy()
    bad[0] ^= 1
    with pytest.raises(yahkv.YahkvError):
        yahkv.slot_check(g, bad)
    # load into a second set of pools, into whatever pages its allocator hands out
    dev2 = yahkv.DevicePools(g, fill=0x77)
    alloc2 = yahkv.PagePool(16)
    alloc2.shuffle(99)
    pages2 = alloc2.alloc(len(pages))
    assert pages2 != pages
    row2 = torch.tensor(pages2, dtype=torch.int32, device="cuda")
    yahkv.slot_unpack(dev2, row2, len(pages2), torch.from_numpy(host).cuda())
    k1, v1 = yahkv.gather_blocks(dev, row, n)
    k2, v2 = yahkv.gather_blocks(dev2, row2, n)
    assert torch.equal(k1, k2) and torch.equal(v1, v2)
    q = torch.randn((1, n_q, hd), device="cuda").to(torch.bfloat16)
    lens = torch.tensor([n], dtype=torch.int32, device="cuda")
    a = yahkv.decode_attend(dev, row[None], lens, n, q, 0.1)
    b = yahkv.decode_attend(dev2, row2[None], lens, n, q, 0.1)
    # same bytes; the waves of a workgroup take tiles in an order that varies from run to run, and with it the running
    # maxima the f16 numerators are rounded against
    assert rel_err(a.cpu().numpy(), b.cpu().numpy()) < 5e-4
    # untouched pages of the second pools keep their fill
    got = dev2.numpy()
    untouched = sorted(set(range(16)) - set(pages2))
    per_page = got["ks"].size // 16
    assert np.all(got["ks"].reshape(16, per_page)[untouched].view(np.uint8) == 0x77)
