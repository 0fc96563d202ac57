"""GPU append fused with RMSNorm + NeoX RoPE (yahkv_append_rope) against the oracle.

Floating point: the rotated rows (K as k_out, Q as q_out) are compared with orc_norm_rope within 1e-3 of the row
maximum for positions below 4096 (f32 angles: position x 2^-24 radians, times the differences between two powf /
sincosf implementations). Bytes: the pools must be bit for bit the oracle's quantization of the kernel's own rotated
rows, placed through the page table, and V must equal the plain append's."""
import numpy as np
import pytest

import oracle
from helpers import bf16_bits, make_tables, rel_err, to_bf16_f32

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.mark.parametrize("fmt,n_q,n_kv,hd,pt,rot,theta,n_new", [
    (8, 24, 4, 256, 64, 256, 1e7, 21), (8, 8, 2, 128, 16, 128, 1e4, 21), (8, 24, 4, 256, 64, 64, 1e6, 21),
    (4, 24, 4, 256, 64, 256, 1e7, 21), (4, 8, 2, 128, 32, 64, 1e4, 21),
    # chunks of eight pages or more: a page's tokens go to the workgroups of one XCD, in another order than the rows'
    (8, 24, 4, 256, 64, 64, 1e6, 600), (4, 8, 2, 128, 16, 128, 1e4, 131), (8, 8, 2, 128, 32, 64, 1e4, 256),
])
def test_fused_append_matches_oracle(yahkv, torch_gpu, fmt, n_q, n_kv, hd, pt, rot, theta, n_new):
    torch = torch_gpu
    rng = np.random.default_rng(fmt * 100 + hd + rot + n_new)
    starts = [0, 37, 1000]
    n_valid = [n_new, 5 if n_new == 21 else n_new - 77, n_new]
    pages = [(s + n_new + pt - 1) // pt for s in starts]
    g = oracle.geometry(fmt, n_q, n_kv, hd, pt, sum(pages) + 1)
    table = make_tables(rng, pages, g.n_pages)
    k = to_bf16_f32(rng.standard_normal((3, n_new, n_kv, hd)) * 3)
    v = to_bf16_f32(rng.standard_normal((3, n_new, n_kv, hd)))
    q = to_bf16_f32(rng.standard_normal((3, n_new, n_q, hd)))
    kw = (1 + 0.2 * rng.standard_normal(hd)).astype(np.float32)
    qw = (1 + 0.2 * rng.standard_normal(hd)).astype(np.float32)
    eps = 1e-6
    to_t = lambda x: torch.from_numpy(bf16_bits(x).view(np.int16)).cuda().view(torch.bfloat16)
    dev = yahkv.DevicePools(yahkv.geometry(fmt, n_q, n_kv, hd, pt, g.n_pages), fill=0x5A)
    t_table = torch.from_numpy(table).cuda()
    t_pos = torch.tensor(starts, dtype=torch.int32, device="cuda")
    t_valid = torch.tensor(n_valid, dtype=torch.int32, device="cuda")
    q_out, k_out = yahkv.append_rope(dev, t_table, t_pos, to_t(k), to_t(v), theta, eps, rot,
                                     k_weight=torch.from_numpy(kw).cuda(), q_weight=torch.from_numpy(qw).cuda(),
                                     q_src=to_t(q), want_k=True, n_valid=t_valid)
    torch.cuda.synchronize()
    q_out, k_out = q_out.cpu().numpy(), k_out.cpu().numpy()
    pos = np.asarray(starts)[:, None] + np.arange(n_new)[None, :]
    want_k = oracle.norm_rope(k, kw, rot, theta, eps, np.broadcast_to(pos[:, :, None], k.shape[:3]))
    want_q = oracle.norm_rope(q, qw, rot, theta, eps, np.broadcast_to(pos[:, :, None], q.shape[:3]))
    for s in range(3):
        nv = n_valid[s]
        assert rel_err(k_out[s, :nv], want_k[s, :nv]) < TOL
        assert rel_err(q_out[s, :nv], want_q[s, :nv]) < TOL
    # bytes: quantize the kernel's own rotated rows with the oracle, through the same table
    host = oracle.HostPools(g, fill=0x5A)
    k_in = np.where((np.arange(n_new)[None, :] < np.asarray(n_valid)[:, None])[:, :, None, None], k_out, 0).astype(np.float32)
    oracle.append(host, table, starts, n_valid, k_in, v)
    got = dev.numpy()
    for name, want in host.arrays().items():
        assert np.array_equal(got[name], want), name
    # V through the plain append gives the same V pools
    plain = yahkv.DevicePools(yahkv.geometry(fmt, n_q, n_kv, hd, pt, g.n_pages), fill=0x5A)
    yahkv.append(plain, t_table, t_pos, to_t(k), to_t(v), n_valid=t_valid)
    p = plain.numpy()
    assert np.array_equal(p["vq"], got["vq"]) and np.array_equal(p["vs"], got["vs"])


def test_fused_append_then_attention_equals_unfused(yahkv, torch_gpu):
    """Rotate on the host, append plainly, attend; against fused append + the same attention: within 2e-3."""
    torch = torch_gpu
    rng = np.random.default_rng(3)
    n_q, n_kv, hd, pt, n = 24, 4, 256, 64, 300
    g = yahkv.geometry(8, n_q, n_kv, hd, pt, 6)
    table = torch.from_numpy(rng.permutation(6).astype(np.int32)[None]).cuda()
    k = rng.standard_normal((1, n, n_kv, hd)).astype(np.float32)
    v = rng.standard_normal((1, n, n_kv, hd)).astype(np.float32)
    q = rng.standard_normal((1, 1, n_q, hd)).astype(np.float32)
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    fused, plain = yahkv.DevicePools(g), yahkv.DevicePools(g)
    yahkv.append_rope(fused, table, zero, torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda(), 1e7, 1e-6, hd)
    # the query of the last position, rotated by a second fused call that appends nothing new of interest
    scratch = yahkv.DevicePools(g)
    q_rot, _ = yahkv.append_rope(scratch, table, zero + (n - 1), torch.from_numpy(k[:, -1:]).cuda(),
                                 torch.from_numpy(v[:, -1:]).cuda(), 1e7, 1e-6, hd, q_src=torch.from_numpy(q).cuda())
    pos = np.arange(n)[None, :, None]
    k_rot = oracle.norm_rope(k, None, hd, 1e7, 1e-6, np.broadcast_to(pos, k.shape[:3]))
    yahkv.append(plain, table, zero, torch.from_numpy(k_rot).cuda(), torch.from_numpy(v).cuda())
    lens = torch.tensor([n], dtype=torch.int32, device="cuda")
    a = yahkv.decode_attend(fused, table, lens, n, q_rot[:, 0].contiguous(), 0.0625).cpu().numpy()
    b = yahkv.decode_attend(plain, table, lens, n, q_rot[:, 0].contiguous(), 0.0625).cpu().numpy()
    assert rel_err(a, b) < 2e-3
    want_q = oracle.norm_rope(q, None, hd, 1e7, 1e-6, np.full((1, 1, n_q), n - 1))
    assert rel_err(q_rot.cpu().numpy(), want_q) < TOL


def test_fused_append_rejects_bad_arguments(yahkv, torch_gpu):
    torch = torch_gpu
    g = yahkv.geometry(8, 8, 2, 128, 16, 4)
    dev = yahkv.DevicePools(g)
    table = torch.zeros((1, 4), dtype=torch.int32, device="cuda")
    zero = torch.zeros(1, dtype=torch.int32, device="cuda")
    k = torch.zeros((1, 2, 2, 128), device="cuda")
    for rot, theta in ((4, 1e4), (12, 1e4), (136, 1e4), (0, 1e4), (128, 0.0)):
        with pytest.raises(yahkv.YahkvError) as e:
            yahkv.append_rope(dev, table, zero, k, k, theta, 1e-6, rot)
        assert e.value.status == -1
