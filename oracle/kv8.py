"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

ctypes binding of the kv8a16 / kv4a16 part of the CPU oracle (oracle/kv8_oracle.c in liboracle.so): the reference's own
KV formats restated on the CPU. Only tests, the smoke check and the benchmark's checks import this module.
"""
import ctypes as C

import numpy as np

from . import lib, _ptr, _i32

HD, PT, TILE = 256, 256, 16          # head_dim, tokens per page, keys per V tile (gen_decode_attn.py:21-27)


class Geometry(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("n_q_heads", "n_kv_heads", "n_pages", "k_bits", "v_bits")]


class Pools(C.Structure):
    _fields_ = [(n, C.c_void_p) for n in ("kq", "ks", "km", "vq", "vs", "vo")]


def geometry(n_q, n_kv, n_pages, k_bits=8, v_bits=8):
    assert k_bits in (4, 8) and v_bits in (4, 8)
    return Geometry(n_q, n_kv, n_pages, k_bits, v_bits)


def quant_k(k, mean):
    """one K row f32 [W] (W a multiple of 128) -> (dwords u32 [W / 4], scale pairs as f16 bits u16 [W / 64])"""
    k = np.ascontiguousarray(k, np.float32).reshape(-1)
    mean = np.ascontiguousarray(mean, np.float32).reshape(-1)
    nh = k.size // 128
    dw, sc = np.zeros(nh * 32, np.uint32), np.zeros(nh * 2, np.uint16)
    lib().orc_kv8_quant_k(_ptr(k), _ptr(mean), C.c_int32(nh), _ptr(dw), _ptr(sc))
    return dw, sc


def deq_k(dw, sc):
    dw, sc = np.ascontiguousarray(dw, np.uint32).reshape(-1), np.ascontiguousarray(sc, np.uint16).reshape(-1)
    nh = sc.size // 2
    out = np.zeros(nh * 128, np.float32)
    lib().orc_kv8_deq_k(_ptr(dw), _ptr(sc), C.c_int32(nh), _ptr(out))
    return out


def quant_vtile(v_bits):
    """v: f16 bits u16 [16][n] -> (dwords u32 [n][4], stats as f16 bits u16 [n][2])"""
    v_bits = np.ascontiguousarray(v_bits, np.uint16)
    n = v_bits.shape[1]
    dw, st = np.zeros((n, 4), np.uint32), np.zeros((n, 2), np.uint16)
    lib().orc_kv8_quant_vtile(_ptr(v_bits), C.c_int32(n), _ptr(dw), _ptr(st))
    return dw, st


def deq_vtile(dw, st):
    dw, st = np.ascontiguousarray(dw, np.uint32), np.ascontiguousarray(st, np.uint16)
    n = dw.shape[0]
    out = np.zeros((16, n), np.float32)
    lib().orc_kv8_deq_vtile(_ptr(dw), _ptr(st), C.c_int32(n), _ptr(out))
    return out


def quant_k4(k, mean):
    """one K row f32 [W] (W a multiple of 256) -> (dwords u32 [W / 8], scale pairs as f16 bits u16 [W / 16])"""
    k = np.ascontiguousarray(k, np.float32).reshape(-1)
    mean = np.ascontiguousarray(mean, np.float32).reshape(-1)
    nh = k.size // 256
    dw, sc = np.zeros(nh * 32, np.uint32), np.zeros(nh * 16, np.uint16)
    lib().orc_kv4_quant_k(_ptr(k), _ptr(mean), C.c_int32(nh), _ptr(dw), _ptr(sc))
    return dw, sc


def deq_k4(dw, sc):
    dw, sc = np.ascontiguousarray(dw, np.uint32).reshape(-1), np.ascontiguousarray(sc, np.uint16).reshape(-1)
    nh = sc.size // 16
    out = np.zeros(nh * 256, np.float32)
    lib().orc_kv4_deq_k(_ptr(dw), _ptr(sc), C.c_int32(nh), _ptr(out))
    return out


def quant_vtile4(v_bits):
    """v: f16 bits u16 [16][n] -> (dwords u32 [n][2], stats as f16 bits u16 [n][2])"""
    v_bits = np.ascontiguousarray(v_bits, np.uint16)
    n = v_bits.shape[1]
    dw, st = np.zeros((n, 2), np.uint32), np.zeros((n, 2), np.uint16)
    lib().orc_kv4_quant_vtile(_ptr(v_bits), C.c_int32(n), _ptr(dw), _ptr(st))
    return dw, st


def deq_vtile4(dw, st):
    dw, st = np.ascontiguousarray(dw, np.uint32), np.ascontiguousarray(st, np.uint16)
    n = dw.shape[0]
    out = np.zeros((16, n), np.float32)
    lib().orc_kv4_deq_vtile(_ptr(dw), _ptr(st), C.c_int32(n), _ptr(out))
    return out


def hadamard256(x):
    """H256 x, unnormalized, f32, in the reference kernels' order of operations; x [..., 256]"""
    x = np.ascontiguousarray(x, np.float32).copy()
    flat = x.reshape(-1, 256)
    for r in flat:
        lib().orc_kv4_hadamard256(_ptr(r))
    return x


def rotate_q(q):
    """q f32 [..., 256] -> H256 q / 16 per head (what the attention over 4-bit K scores against)"""
    q = np.ascontiguousarray(q, np.float32)
    out = np.zeros_like(q)
    qf, of = q.reshape(-1, 256), out.reshape(-1, 256)
    for i in range(qf.shape[0]):
        lib().orc_kv4_rotate_q(_ptr(qf[i]), _ptr(of[i]))
    return out


def kmean(k):
    """k f32 [n_rows][W] -> per-channel mean f32 [W] of the f16-truncated rows"""
    k = np.ascontiguousarray(k, np.float32)
    mean = np.zeros(k.shape[1], np.float32)
    lib().orc_kv8_kmean(_ptr(k), C.c_int32(k.shape[0]), C.c_int32(k.shape[1]), _ptr(mean))
    return mean


class HostPools:
    """The six buffers of one layer in host memory, in the reference's layouts (see kv8_oracle.h)."""

    NAMES = ("kq", "ks", "km", "vq", "vs", "vo")

    def __init__(self, geom, fill=0):
        self.geom = geom
        H, P = geom.n_kv_heads, geom.n_pages
        W = H * HD
        f = np.uint32(fill * 0x01010101)
        self.kq = np.full((P * PT, W // (8 if geom.k_bits == 4 else 4)), f, np.uint32)
        self.ks = np.full((P * PT, W // (32 if geom.k_bits == 4 else 128)), f, np.uint32)
        self.km = np.full((P, W), f, np.uint32).view(np.float32)
        self.vq = np.full((H, P * 16, HD, 2 if geom.v_bits == 4 else 4), f, np.uint32)
        self.vs = np.full((H, P * 16, HD), f, np.uint32)
        self.vo = np.full((P, W, 16), np.uint16(fill * 257), np.uint16)

    def struct(self):
        return Pools(*[getattr(self, n).ctypes.data for n in self.NAMES])

    def arrays(self):
        return {n: getattr(self, n) for n in self.NAMES}


def append(pools, table, start_pos, n_valid, k_src, v_src):
    """k_src / v_src: f32 [n_seqs][n_new][W]."""
    table, start_pos, n_valid = _i32(table), _i32(start_pos), _i32(n_valid)
    k_src, v_src = np.ascontiguousarray(k_src, np.float32), np.ascontiguousarray(v_src, np.float32)
    st = pools.struct()
    lib().orc_kv8_append(C.byref(pools.geom), C.byref(st), _ptr(table), C.c_int32(table.shape[1]), _ptr(start_pos),
                         _ptr(n_valid), C.c_int32(k_src.shape[0]), C.c_int32(k_src.shape[1]), _ptr(k_src), _ptr(v_src))


def dense(pools, table_row, n_tokens, as_f16=False):
    """(Kd, Vd) f32 [n_tokens][H][256]: the sequence's first n_tokens as the decode attention sees them (K - mean;
    closed V tiles from codes, the newest from the open tile), or, as_f16, as the prefill attention does."""
    g = pools.geom
    W = g.n_kv_heads * HD
    row = _i32(table_row)
    Kd, Vd = np.zeros((n_tokens, W), np.float32), np.zeros((n_tokens, W), np.float32)
    st = pools.struct()
    fn = lib().orc_kv8_dense_f16 if as_f16 else lib().orc_kv8_dense
    fn(C.byref(g), C.byref(st), _ptr(row), C.c_int32(n_tokens), _ptr(Kd), _ptr(Vd))
    return Kd.reshape(n_tokens, g.n_kv_heads, HD), Vd.reshape(n_tokens, g.n_kv_heads, HD)


def pools_of_sequence(dev, table_row, n_tokens):
    """The pages of one sequence, copied from device pools (an object with uint8 torch tensors kq, ks, km, vq, vs, vopen
    and a geometry) into host pools of their own, numbered in logical order: (HostPools, identity table row)."""
    g = dev.geom
    H, W = g.n_kv_heads, g.n_kv_heads * HD
    n_pg = max((n_tokens + PT - 1) // PT, 1)
    import torch
    pg = torch.as_tensor(np.asarray(table_row[:n_pg], np.int64), device=dev.kq.device)
    kb, vb = getattr(dev, "k_bits", 8), getattr(dev, "v_bits", 8)
    hp = HostPools(geometry(g.n_q_heads, H, n_pg, kb, vb))
    take = lambda t, shape: t.view(*shape)
    kqw, ksw, vqw = hp.kq.shape[1], hp.ks.shape[1], hp.vq.shape[3]
    hp.kq[:] = take(dev.kq, (g.n_pages, PT * kqw * 4))[pg].cpu().numpy().view(np.uint32).reshape(n_pg * PT, kqw)
    hp.ks[:] = take(dev.ks, (g.n_pages, PT * ksw * 4))[pg].cpu().numpy().view(np.uint32).reshape(n_pg * PT, ksw)
    hp.km[:] = take(dev.km, (g.n_pages, W * 4))[pg].cpu().numpy().view(np.float32).reshape(n_pg, W)
    hp.vq[:] = take(dev.vq, (H, g.n_pages, 16 * HD * vqw * 4))[:, pg].cpu().numpy().view(np.uint32).reshape(H, n_pg * 16, HD, vqw)
    hp.vs[:] = take(dev.vs, (H, g.n_pages, 16 * HD * 4))[:, pg].cpu().numpy().view(np.uint32).reshape(H, n_pg * 16, HD)
    hp.vo[:] = take(dev.vopen, (g.n_pages, W * 16 * 2))[pg].cpu().numpy().view(np.uint16).reshape(n_pg, W, 16)
    return hp, np.arange(n_pg, dtype=np.int32)
