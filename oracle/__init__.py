"""TEST INFRASTRUCTURE, NOT PRODUCT CODE.

ctypes binding of the CPU oracle (oracle/liboracle.so, built from yahkv_oracle.c) and, where it was built, of
the reference's own block quantizer (oracle/_ref/libref.so). Only tests, the smoke check and the benchmark's
CPU-baseline leg import this module; the library under test never does.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "liboracle.so")
REF = os.path.join(HERE, "_ref", "libref.so")


def build():
    """Compile liboracle.so and, if the reference tree is present, _ref/libref.so."""
    subprocess.run(["make", "-C", HERE, "-B", "all"], check=True, capture_output=True)


class Geometry(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("format", "n_q_heads", "n_kv_heads", "head_dim", "page_tokens", "n_pages")]


class Pools(C.Structure):
    _fields_ = [("kq", C.c_void_p), ("ks", C.c_void_p), ("vq", C.c_void_p), ("vs", C.c_void_p)]


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


_lib = None
_ref = None


def lib(path=None):
    global _lib
    if _lib is None:
        if path is None and not os.path.exists(LIB):
            build()
        _lib = C.CDLL(path or LIB)
        for n in ("orc_kq_bytes", "orc_ks_bytes", "orc_vq_bytes", "orc_vs_bytes"):
            getattr(_lib, n).restype = C.c_size_t
            getattr(_lib, n).argtypes = [C.POINTER(Geometry)]
        _lib.orc_threads.restype = C.c_int32
        _lib.orc_lround_identity_mismatches.restype = C.c_uint64
        _lib.orc_lround_identity_mismatches.argtypes = [C.c_uint32, C.c_uint32]
    return _lib


def use_native_build():
    """For the benchmark's CPU-baseline leg: compile the oracle again for this machine's own host cores with the
    reference's host flags (-O3 -march=native -ffp-contract=off, engine/build_hrx.sh:26) and use that library from now
    on. The committed build recipe leaves -march out so that the library runs on whatever box it is carried to; a
    native build cannot travel. Falls back to the portable library if no compiler is here. Returns the flags in use."""
    global _lib
    import tempfile
    out = os.path.join(tempfile.gettempdir(), f"liboracle_native_{os.getpid()}.so")
    flags = ["-std=c11", "-O3", "-march=native", "-ffp-contract=off", "-fopenmp", "-fPIC", "-shared"]
    try:
        subprocess.run(["gcc"] + flags + ["-o", out, os.path.join(HERE, "yahkv_oracle.c"),
                        os.path.join(HERE, "kv8_oracle.c"), "-lm"], check=True,
                       capture_output=True, timeout=120)
    except (OSError, subprocess.SubprocessError):
        lib()
        return "gcc -O3 -ffp-contract=off -fopenmp (portable build: no compiler on this box for -march=native)"
    _lib = None
    lib(out)
    os.unlink(out)                                            # the mapping stays; the file need not
    return "gcc " + " ".join(flags[1:5])


def ref():
    """The reference's compiled block code, or None if oracle/_ref was not built."""
    global _ref
    if _ref is None and os.path.exists(REF):
        _ref = C.CDLL(REF)
    return _ref


def _blocks(fn, x, bb):
    x = np.ascontiguousarray(x, np.float32).reshape(-1)
    assert x.size % 32 == 0
    out = np.zeros(x.size // 32 * bb, np.uint8)
    fn(_ptr(x), C.c_uint64(x.size), _ptr(out))
    return out.reshape(-1, bb)


def _deq(fn, blocks, bb):
    blocks = np.ascontiguousarray(blocks, np.uint8).reshape(-1, bb)
    out = np.zeros(blocks.shape[0] * 32, np.float32)
    fn(_ptr(blocks), C.c_uint64(out.size), _ptr(out))
    return out


def quantize_q8_0(x):
    return _blocks(lib().orc_quantize_q8_0, x, 34)


def quantize_q4_0(x):
    return _blocks(lib().orc_quantize_q4_0, x, 18)


def dequantize_q8_0(b):
    return _deq(lib().orc_dequantize_q8_0, b, 34)


def dequantize_q4_0(b):
    return _deq(lib().orc_dequantize_q4_0, b, 18)


def ref_quantize_q8_0(x):
    return _blocks(ref().ref_quantize_q8_0, x, 34)


def ref_dequantize_q8_0(b):
    return _deq(ref().ref_dequantize_q8_0, b, 34)


def ref_dequantize_q4_0(b):
    return _deq(ref().ref_dequantize_q4_0, b, 18)


def _conv(fn, x, src, dst):
    x = np.ascontiguousarray(x, src).reshape(-1)
    y = np.zeros(x.size, dst)
    fn(_ptr(x), C.c_uint64(x.size), _ptr(y))
    return y


def f32_to_f16_bits(x):
    return _conv(lib().orc_f32_to_f16_n, x, np.float32, np.uint16)


def f16_bits_to_f32(x):
    return _conv(lib().orc_f16_to_f32_n, x, np.uint16, np.float32)


def f32_to_bf16_bits(x):
    return _conv(lib().orc_f32_to_bf16_n, x, np.float32, np.uint16)


def bf16_bits_to_f32(x):
    return _conv(lib().orc_bf16_to_f32_n, x, np.uint16, np.float32)


def ref_f16_bits_to_f32(x):
    return _conv(ref().ref_f16_to_f32, x, np.uint16, np.float32)


def ref_bf16_bits_to_f32(x):
    return _conv(ref().ref_bf16_to_f32, x, np.uint16, np.float32)


class HostPools:
    """The four pools of one layer in host memory, in the library's page layout."""

    def __init__(self, geom, fill=0):
        self.geom = geom
        g = C.byref(geom)
        L = lib()
        self.kq = np.full(L.orc_kq_bytes(g), fill, np.uint8)
        self.ks = np.full(L.orc_ks_bytes(g) // 2, fill * 257, np.uint16)
        self.vq = np.full(L.orc_vq_bytes(g), fill, np.uint8)
        self.vs = np.full(L.orc_vs_bytes(g) // 2, fill * 257, np.uint16)

    def struct(self):
        return Pools(self.kq.ctypes.data, self.ks.ctypes.data, self.vq.ctypes.data, self.vs.ctypes.data)

    def arrays(self):
        return {"kq": self.kq, "ks": self.ks, "vq": self.vq, "vs": self.vs}


def geometry(fmt, n_q, n_kv, head_dim, page_tokens, n_pages):
    return Geometry(fmt, n_q, n_kv, head_dim, page_tokens, n_pages)


def _i32(a):
    return None if a is None else np.ascontiguousarray(a, np.int32)


def append(pools, table, start_pos, n_valid, k_src, v_src):
    """k_src / v_src: f32 [n_seqs][n_new][H][D]."""
    table = _i32(table)
    start_pos, n_valid = _i32(start_pos), _i32(n_valid)
    k_src = np.ascontiguousarray(k_src, np.float32)
    v_src = np.ascontiguousarray(v_src, np.float32)
    n_seqs, n_new = k_src.shape[0], k_src.shape[1]
    st = pools.struct()
    lib().orc_append(C.byref(pools.geom), C.byref(st), _ptr(table), C.c_int32(table.shape[1]), _ptr(start_pos),
                     _ptr(n_valid), C.c_int32(n_seqs), C.c_int32(n_new), _ptr(k_src), _ptr(v_src))


def norm_rope(x, weight, rotary_dim, theta, eps, pos):
    """x f32 [..., D] rows; pos int per row (same leading shape); returns the normalised, rotated rows."""
    x = np.ascontiguousarray(x, np.float32)
    d = x.shape[-1]
    rows = x.reshape(-1, d)
    pos = np.ascontiguousarray(np.broadcast_to(np.asarray(pos, np.int32), x.shape[:-1]).reshape(-1), np.int32)
    w = None if weight is None else np.ascontiguousarray(weight, np.float32)
    out = np.empty_like(rows)
    lib().orc_norm_rope(_ptr(rows), _ptr(w), C.c_int32(rows.shape[0]), C.c_int32(d), C.c_int32(rotary_dim),
                        C.c_float(theta), C.c_float(eps), _ptr(pos), _ptr(out))
    return out.reshape(x.shape)


def gather_blocks(pools, table_row, n_tokens):
    g = pools.geom
    bb = 34 if g.format == 8 else 18
    shape = (n_tokens, g.n_kv_heads, g.head_dim // 32, bb)
    k = np.zeros(shape, np.uint8)
    v = np.zeros(shape, np.uint8)
    st = pools.struct()
    row = _i32(table_row)
    lib().orc_gather_blocks(C.byref(g), C.byref(st), _ptr(row), C.c_int32(n_tokens), _ptr(k), _ptr(v))
    return k, v


def decode_attend(pools, table, seq_len, q, scale, gate=None):
    g = pools.geom
    table, seq_len = _i32(table), _i32(seq_len)
    q = np.ascontiguousarray(q, np.float32)
    gate = None if gate is None else np.ascontiguousarray(gate, np.float32)
    out = np.zeros(q.shape, np.float32)
    st = pools.struct()
    lib().orc_decode_attend(C.byref(g), C.byref(st), _ptr(table), C.c_int32(table.shape[1]), _ptr(seq_len),
                            C.c_int32(len(seq_len)), _ptr(q), C.c_float(scale), _ptr(gate), _ptr(out))
    return out


def prefill_attend(pools, table, prefix_len, q, scale, gate=None):
    """q f32 [n_seqs][chunk_len][n_q_heads][D]."""
    g = pools.geom
    table, prefix_len = _i32(table), _i32(prefix_len)
    q = np.ascontiguousarray(q, np.float32)
    gate = None if gate is None else np.ascontiguousarray(gate, np.float32)
    out = np.zeros(q.shape, np.float32)
    st = pools.struct()
    lib().orc_prefill_attend(C.byref(g), C.byref(st), _ptr(table), C.c_int32(table.shape[1]), _ptr(prefix_len),
                             C.c_int32(q.shape[0]), C.c_int32(q.shape[1]), _ptr(q), C.c_float(scale), _ptr(gate),
                             _ptr(out))
    return out


def threads():
    return int(lib().orc_threads())


def lround_identity_mismatches(first_bits, last_bits):
    """Floats (both signs) with magnitude bits in [first_bits, last_bits] for which lroundf(r) differs from the
    truncation of r + copysignf(0.5 - 2^-25, r), the form the append kernels compute."""
    return int(lib().orc_lround_identity_mismatches(first_bits, last_bits))
