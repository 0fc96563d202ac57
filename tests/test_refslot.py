"""The reader for the reference's own slot files ("YAHSLOT1", LoomPrefill::SaveState / LoadState,
engine/model/loom_prefill.hpp:976-1024). The reference tree holds no slot file (they are written on the reference's own
machine from a model's prefill), so the files here are written by this test in the layout SaveState's code writes: five
u64 {magic, T, B, chunks, 10}, then per buffer a u64 length and the raw bytes, in the order of StateBuffers()
(:1027-1030), the KV buffers holding every full-attention layer one after the other (DecoderState(), :952-972). Parity
unpinned against a file of the reference's making; pinned against that code's reading."""
import struct

import numpy as np
import pytest

import kv8_recipe
from helpers import closed_form, rel_err
from oracle import kv8

MAGIC = 0x31544F4C53484159          # "YAHSLOT1", loom_prefill.hpp:1025


def slot_file(layers, ptab, T, B, chunks, conv=b"\x01" * 100, state=b"\x02" * 52):
    """layers: oracle HostPools of one sequence each (the reference's single-sequence pools, n_pages = T / 256)."""
    cat = lambda name: b"".join(np.ascontiguousarray(getattr(hp, name)).tobytes() for hp in layers)
    km = b"".join(np.ascontiguousarray(hp.km[ptab[0]]).tobytes() for hp in layers)   # one mean vector per layer (:958)
    bufs = [np.asarray(ptab, np.int32).tobytes(), cat("kq"), cat("ks"), km, cat("vq"), cat("vs"), b"", b"", conv, state]
    out = struct.pack("<5Q", MAGIC, T, B, chunks, len(bufs))
    for b in bufs:
        out += struct.pack("<Q", len(b)) + b
    return out


def layers_of(rc, n_tokens, kb, vb, n_layers=2):
    out = []
    for li in range(n_layers):
        hp = kv8.HostPools(kv8.geometry(24, 4, rc.T // 256, kb, vb), 0)
        hp.km[rc.ptab[0]] = rc.m * (li + 1)
        K = (rc.K.astype(np.float32) * (1 + 0.25 * li))[None, :n_tokens]
        kv8.append(hp, rc.ptab[None], [0], None, K, np.roll(rc.V.astype(np.float32), li, 1)[None, :n_tokens])
        out.append(hp)
    return out


@pytest.fixture(scope="module")
def rc():
    return kv8_recipe.load(8)


@pytest.mark.parametrize("kb,vb,fmt", [(8, 8, 816), (4, 4, 416), (8, 4, 8416), (4, 8, 4816)])
def test_parse_reports_what_the_file_holds(yahkv, rc, kb, vb, fmt):
    f = slot_file(layers_of(rc, 512, kb, vb, 3), rc.ptab, 1024, 256, 2)
    info = yahkv.refslot_parse(f)
    assert (info.context, info.chunk, info.chunks) == (1024, 256, 2)
    assert (info.n_pages, info.n_layers, info.n_kv_heads, info.format) == (4, 3, 4, fmt)
    assert info.size[0] == 16 and info.offset[0] == 48
    assert info.size[3] == 3 * 4096 and info.size[8] == 100 and info.size[9] == 52
    assert info.offset[9] + info.size[9] == len(f)


def test_parse_refuses_what_loadstate_would(yahkv, rc):
    good = slot_file(layers_of(rc, 256, 8, 8, 1), rc.ptab, 1024, 256, 1)
    yahkv.refslot_parse(good)
    bad = [b"YAHSLOT2" + good[8:],                               # another magic
           good[:len(good) - 10],                                # truncated in the last buffer
           good[:44],                                            # truncated in a length
           good[:32] + struct.pack("<Q", 9) + good[40:],         # another number of state buffers (:1008)
           good[:24] + struct.pack("<Q", 5) + good[32:]]         # more chunks than the context holds
    p = bytearray(good)
    p[48:52] = struct.pack("<i", 4)                              # a page table entry outside the pool
    bad.append(bytes(p))
    half = layers_of(rc, 256, 8, 8, 1)
    half[0].ks = half[0].ks[:, :4]                               # scales that fit no format
    bad.append(slot_file(half, rc.ptab, 1024, 256, 1))
    for i, f in enumerate(bad):
        with pytest.raises(yahkv.YahkvError):
            yahkv.refslot_parse(f)
            pytest.fail(f"case {i} was accepted")


@pytest.mark.gpu
@pytest.mark.parametrize("kb,vb", [(8, 8), (4, 4)])
def test_a_layer_loads_into_other_pages_and_attends_alike(yahkv, torch_gpu, rc, kb, vb):
    """A two-layer slot covering 512 tokens: layer 1 loaded into pages (5, 2) of a six-page pool gives the bytes the
    oracle's pools hold, page for page, and the decode attention over them equals the closed form over the oracle's
    model of the original pools; then decode steps continue from there."""
    torch = torch_gpu
    n = 512
    layers = layers_of(rc, n, kb, vb)
    f = np.frombuffer(slot_file(layers, rc.ptab, 1024, 256, 2), np.uint8)
    g = yahkv.kv8_geometry(24, 4, 6, kb, vb)
    dp = yahkv.Kv8Pools(g, 0x5A)
    mine = [5, 2, 0]
    yahkv.refslot_load_layer(dp, f, 1, mine)
    got, src = dp.numpy(), layers[1]
    for lp in range(2):
        a, b = mine[lp], int(rc.ptab[lp])
        assert np.array_equal(got["kq"][a * 256:a * 256 + 256], src.kq[b * 256:b * 256 + 256])
        assert np.array_equal(got["ks"][a * 256:a * 256 + 256], src.ks[b * 256:b * 256 + 256])
        assert np.array_equal(got["vq"][:, a * 16:a * 16 + 16], src.vq[:, b * 16:b * 16 + 16])
        assert np.array_equal(got["vs"][:, a * 16:a * 16 + 16], src.vs[:, b * 16:b * 16 + 16])
    assert np.array_equal(got["km"][5], src.km[rc.ptab[0]])
    for untouched in (0, 1, 3, 4):
        assert np.all(got["kq"][untouched * 256:untouched * 256 + 256] == 0x5A5A5A5A)
        assert np.all(got["vq"][:, untouched * 16:untouched * 16 + 16] == 0x5A5A5A5A)
    table = torch.tensor([mine], dtype=torch.int32, device="cuda")
    q = torch.from_numpy(rc.q[None]).cuda()
    # A slot ends on a whole chunk, so on a tile boundary, and does not carry the open tile: what follows is a decode
    # step (loom_decoder.hpp:233-235), which reads every tile of the slot from its codes and opens a new one.
    kn = torch.from_numpy(rc.K[n].astype(np.float32).reshape(1, 4, 256) * 1.25).cuda()
    vn = torch.from_numpy(np.roll(rc.V.astype(np.float32), 1, 1)[n].reshape(1, 4, 256)).cuda()
    out = yahkv.kv8_decode_step(dp, table, torch.tensor([n + 1], dtype=torch.int32, device="cuda"), n + 1, kn, vn, q, 1.0 / 16.0)
    want_pools = layers_of(rc, n + 1, kb, vb)[1]      # the oracle's pools of the same layer after the same 513 tokens
    Kd, Vd = kv8.dense(want_pools, rc.ptab, n + 1)
    qx = kv8.rotate_q(rc.q) if kb == 4 else rc.q
    assert rel_err(out.cpu().numpy()[0], closed_form(Kd, Vd, qx, 1.0 / 16.0)) < 2e-3
