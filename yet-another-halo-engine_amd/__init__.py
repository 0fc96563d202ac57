"""Python binding of libyahkv.so (the C ABI of include/yahkv.h) for tests and benchmarks.

PyTorch only provides device memory and streams here: every call passes raw device pointers and torch's current HIP
stream to the library. There is no CPU fallback: without the built library the import fails.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libyahkv.so")

Q8_0, Q4_0, KV_F16, KV8A16 = 8, 4, 16, 816
KV4A16, K8V4A16, K4V8A16 = 416, 8416, 4816
_KV8_FORMATS = {(8, 8): KV8A16, (4, 4): KV4A16, (8, 4): K8V4A16, (4, 8): K4V8A16}
F32, F16, BF16 = 0, 1, 2


class YahkvError(RuntimeError):
    def __init__(self, status, what):
        super().__init__(f"{what}: {status_text(status)} ({status})")
        self.status = status


class Geometry(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("format", "n_q_heads", "n_kv_heads", "head_dim", "page_tokens", "n_pages")]


class Pools(C.Structure):
    _fields_ = [("kq", C.c_void_p), ("ks", C.c_void_p), ("vq", C.c_void_p), ("vs", C.c_void_p),
                ("kq_bytes", C.c_size_t), ("ks_bytes", C.c_size_t), ("vq_bytes", C.c_size_t), ("vs_bytes", C.c_size_t)]


class F16PoolsStruct(C.Structure):
    _fields_ = [("k", C.c_void_p), ("v", C.c_void_p), ("k_bytes", C.c_size_t), ("v_bytes", C.c_size_t)]


class Kv8PoolsStruct(C.Structure):
    _NAMES = ("kq", "ks", "km", "vq", "vs", "vopen")
    _fields_ = [(n, C.c_void_p) for n in _NAMES] + [(n + "_bytes", C.c_size_t) for n in _NAMES]


class DecodeOptions(C.Structure):
    """yahkv_decode_options: zero fields are the defaults."""
    _fields_ = [("n_chunks", C.c_int32), ("min_chunk_tiles", C.c_int32), ("pair_cost", C.c_int32),
                ("reduce_split", C.c_int32), ("deterministic", C.c_int32), ("xcd_weight", C.c_int32 * 8),
                ("one_launch", C.c_int32), ("wg_partials", C.c_int32), ("cut", C.c_int32)]


class Rope(C.Structure):
    _fields_ = [("theta", C.c_float), ("eps", C.c_float), ("rotary_dim", C.c_int32), ("k_weight", C.c_void_p),
                ("q_weight", C.c_void_p)]


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is not built: run `python __graft_entry__.py build` (hipcc, gfx950)")
    # torch ships its own HIP runtime (same soname as /opt/rocm's). It must be in the process first, so that the
    # library binds to that one: two runtimes in one process do not share streams or device memory.
    import torch  # noqa: F401
    lib = C.CDLL(LIB_PATH)
    G, P, vp, i32, i32p = C.POINTER(Geometry), C.POINTER(Pools), C.c_void_p, C.c_int32, C.c_void_p
    lib.yahkv_version.restype = C.c_char_p
    lib.yahkv_strerror.restype = C.c_char_p
    lib.yahkv_strerror.argtypes = [C.c_int]
    lib.yahkv_check_geometry.argtypes = [G]
    for n in ("yahkv_kq_bytes", "yahkv_ks_bytes", "yahkv_vq_bytes", "yahkv_vs_bytes", "yahkv_bytes_per_token"):
        getattr(lib, n).restype = C.c_size_t
        getattr(lib, n).argtypes = [G]
    lib.yahkv_validate_page_table.argtypes = [G, i32p, i32, i32p, i32]
    lib.yahkv_append.argtypes = [G, P, i32p, i32, i32p, i32p, i32, i32, vp, vp, i32, vp]
    lib.yahkv_append_rope.argtypes = [G, P, i32p, i32, i32p, i32p, i32, i32, vp, vp, i32, C.POINTER(Rope), vp, vp, i32,
                                      vp, vp]
    lib.yahkv_decode_workspace_bytes.restype = C.c_size_t
    O = C.POINTER(DecodeOptions)
    lib.yahkv_decode_workspace_bytes.argtypes = [G, i32, i32, O]
    lib.yahkv_decode_workspace_init.argtypes = [G, i32, i32, O, vp, C.c_size_t, vp]
    lib.yahkv_decode_part.argtypes = [G, P, i32p, i32, i32p, i32, i32, vp, i32, C.c_float, vp, C.c_size_t, O, vp]
    lib.yahkv_decode_reduce.argtypes = [G, i32, i32p, i32, i32, vp, vp, vp, C.c_size_t, O, vp]
    lib.yahkv_decode_attend.argtypes = [G, P, i32p, i32, i32p, i32, i32, vp, i32, C.c_float, vp, vp, vp, C.c_size_t, O,
                                        vp]
    lib.yahkv_decode_step.argtypes = [G, P, i32p, i32, i32p, i32, i32, vp, vp, i32, vp, i32, C.c_float, vp, vp, vp,
                                      C.c_size_t, O, vp]
    lib.yahkv_decode_step_reduce.argtypes = lib.yahkv_decode_step.argtypes
    lib.yahkv_decode_calibrate.argtypes = [G, P, i32p, i32, i32p, i32, i32, vp, i32, vp, C.c_size_t, O, i32, vp]
    lib.yahkv_shader_clock_probe.argtypes = [vp, i32, vp]
    lib.yahkv_decode_static_scratch_bytes.restype = C.c_size_t
    lib.yahkv_decode_attend_static.argtypes = [G, P, i32p, i32, i32p, i32, i32, vp, i32, C.c_float, vp, vp, vp]
    lib.yahkv_prefill_workspace_bytes.restype = C.c_size_t
    lib.yahkv_prefill_workspace_bytes.argtypes = [G, i32, i32, i32]
    lib.yahkv_prefill_attend.argtypes = [G, P, i32p, i32, i32p, i32, i32, i32, vp, C.c_float, vp, vp, i32, vp,
                                         C.c_size_t, vp]
    lib.yahkv_prefill_attend_tiles.argtypes = lib.yahkv_prefill_attend.argtypes
    F = C.POINTER(F16PoolsStruct)
    lib.yahkv_f16_pool_bytes.restype = C.c_size_t
    lib.yahkv_f16_pool_bytes.argtypes = [G]
    lib.yahkv_f16_append.argtypes = [G, F, i32p, i32, i32p, i32p, i32, i32, vp, vp, i32, vp]
    lib.yahkv_f16_prefill_workspace_bytes.restype = C.c_size_t
    lib.yahkv_f16_prefill_workspace_bytes.argtypes = [G, i32, i32, i32]
    lib.yahkv_f16_prefill_attend.argtypes = [G, F, i32p, i32, i32p, i32, i32, i32, vp, C.c_float, vp, vp, i32, vp,
                                             C.c_size_t, vp]
    lib.yahkv_f16_decode_workspace_bytes.restype = C.c_size_t
    lib.yahkv_f16_decode_workspace_bytes.argtypes = [G, i32, i32, O]
    lib.yahkv_f16_decode_attend.argtypes = [G, F, i32p, i32, i32p, i32, i32, vp, i32, C.c_float, vp, vp, vp,
                                            C.c_size_t, O, vp]
    lib.yahkv_prefill_decode_tiles.argtypes = [G, P, i32p, i32, i32p, i32, i32, i32, vp, C.c_size_t, vp]
    K8 = C.POINTER(Kv8PoolsStruct)
    for n in Kv8PoolsStruct._NAMES:
        getattr(lib, f"yahkv_kv8_{n}_bytes").restype = C.c_size_t
        getattr(lib, f"yahkv_kv8_{n}_bytes").argtypes = [G]
    lib.yahkv_kv8_kmean.argtypes = [G, K8, i32p, i32, i32p, i32, i32, vp, i32, vp]
    lib.yahkv_kv8_append.argtypes = [G, K8, i32p, i32, i32p, i32p, i32, i32, vp, vp, i32, vp]
    lib.yahkv_kv8_decode_workspace_bytes.restype = C.c_size_t
    lib.yahkv_kv8_decode_workspace_bytes.argtypes = [G, i32, i32, O]
    lib.yahkv_kv8_decode_attend.argtypes = [G, K8, i32p, i32, i32p, i32, i32, vp, i32, C.c_float, vp, vp, vp, C.c_size_t,
                                            O, vp]
    lib.yahkv_kv8_decode_part.argtypes = [G, K8, i32p, i32, i32p, i32, i32, vp, i32, C.c_float, vp, C.c_size_t, O, vp]
    lib.yahkv_kv8_decode_reduce.argtypes = [G, K8, i32p, i32, i32p, i32, i32, vp, vp, i32, vp, i32, C.c_float, vp, vp,
                                            vp, C.c_size_t, O, vp]
    lib.yahkv_kv8_slot_bytes.restype = C.c_size_t
    lib.yahkv_kv8_slot_bytes.argtypes = [G, i32]
    lib.yahkv_kv8_prefill_workspace_bytes.restype = C.c_size_t
    lib.yahkv_kv8_prefill_workspace_bytes.argtypes = [G, i32, i32, i32]
    lib.yahkv_kv8_prefill_attend.argtypes = [G, K8, i32p, i32, i32p, i32, i32, i32, vp, C.c_float, vp, vp, i32, vp,
                                             C.c_size_t, vp]
    lib.yahkv_kv8_decode_step.argtypes = [G, K8, i32p, i32, i32p, i32, i32, vp, vp, i32, vp, i32, C.c_float, vp, vp, vp,
                                          C.c_size_t, O, vp]
    lib.yahkv_gather_blocks.argtypes = [G, P, i32p, i32, vp, vp, vp]
    lib.yahkv_pagepool_create.restype = C.c_void_p
    lib.yahkv_pagepool_create.argtypes = [i32]
    lib.yahkv_pagepool_destroy.argtypes = [vp]
    lib.yahkv_pagepool_free_count.argtypes = [vp]
    lib.yahkv_pagepool_alloc.argtypes = [vp, i32, i32p]
    lib.yahkv_pagepool_free.argtypes = [vp, i32p, i32]
    lib.yahkv_pagepool_shuffle.argtypes = [vp, C.c_uint64]
    lib.yahkv_pagepool_retain.argtypes = [vp, i32p, i32]
    lib.yahkv_pagepool_refcount.argtypes = [vp, i32]
    lib.yahkv_copy_pages.argtypes = [G, P, i32p, i32p, i32, vp]
    lib.yahkv_slot_bytes.restype = C.c_size_t
    lib.yahkv_slot_bytes.argtypes = [G, i32]
    lib.yahkv_slot_pack.argtypes = [G, P, i32p, i32, i32, vp, vp]
    lib.yahkv_slot_check.argtypes = [G, vp, C.c_size_t, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
    lib.yahkv_slot_unpack.argtypes = [G, P, i32p, i32, vp, vp]
    return lib


lib = _load()


def status_text(status):
    return lib.yahkv_strerror(int(status)).decode()


def _check(status, what):
    if status != 0:
        raise YahkvError(status, what)


def geometry(fmt, n_q_heads, n_kv_heads, head_dim, page_tokens, n_pages):
    g = Geometry(fmt, n_q_heads, n_kv_heads, head_dim, page_tokens, n_pages)
    _check(lib.yahkv_check_geometry(C.byref(g)), "geometry")
    return g


def pool_bytes(g):
    r = C.byref(g)
    return {"kq": lib.yahkv_kq_bytes(r), "ks": lib.yahkv_ks_bytes(r), "vq": lib.yahkv_vq_bytes(r),
            "vs": lib.yahkv_vs_bytes(r)}


def validate_page_table(g, table, seq_len):
    """table: numpy int32 [n_seqs][stride]; seq_len: numpy int32 [n_seqs]. Raises YahkvError on a bad table."""
    import numpy as np
    table = np.ascontiguousarray(table, np.int32)
    seq_len = np.ascontiguousarray(seq_len, np.int32)
    _check(lib.yahkv_validate_page_table(C.byref(g), table.ctypes.data, table.shape[1], seq_len.ctypes.data,
                                         len(seq_len)), "page table")


class PagePool:
    """Host page allocator with a free list (yahkv_pagepool_*)."""

    def __init__(self, n_pages):
        self._p = lib.yahkv_pagepool_create(n_pages)
        if not self._p:
            raise YahkvError(-1, "pagepool_create")

    def close(self):
        if self._p:
            lib.yahkv_pagepool_destroy(self._p)
            self._p = None

    __del__ = close

    @property
    def free_count(self):
        return lib.yahkv_pagepool_free_count(self._p)

    def alloc(self, n):
        out = (C.c_int32 * max(n, 1))()
        _check(lib.yahkv_pagepool_alloc(self._p, n, C.cast(out, C.c_void_p)), "pagepool_alloc")
        return list(out[:n])

    def free(self, pages):
        arr = (C.c_int32 * max(len(pages), 1))(*pages)
        _check(lib.yahkv_pagepool_free(self._p, C.cast(arr, C.c_void_p), len(pages)), "pagepool_free")

    def shuffle(self, seed):
        lib.yahkv_pagepool_shuffle(self._p, seed)

    def retain(self, pages):
        arr = (C.c_int32 * max(len(pages), 1))(*pages)
        _check(lib.yahkv_pagepool_retain(self._p, C.cast(arr, C.c_void_p), len(pages)), "pagepool_retain")

    def refcount(self, page):
        return lib.yahkv_pagepool_refcount(self._p, page)


# ---- device side (torch supplies memory and the stream) --------------------------------------------------------------

def _stream():
    import torch
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _dp(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _dtype_code(t):
    import torch
    return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[t.dtype]


class F16Pools:
    """One layer's unquantized f16 K and V^T pools on the GPU (the reference's kpool / vtpool of the fp16 kernels)."""

    def __init__(self, g, fill=0, device="cuda:0"):
        import torch
        assert g.format == KV_F16
        self.geom = g
        n = lib.yahkv_f16_pool_bytes(C.byref(g))
        if n == 0:
            raise YahkvError(-2, "f16 pools")
        self.k = torch.full((n,), fill, dtype=torch.uint8, device=device)
        self.v = torch.full((n,), fill, dtype=torch.uint8, device=device)

    def struct(self):
        return F16PoolsStruct(self.k.data_ptr(), self.v.data_ptr(), self.k.numel(), self.v.numel())

    def numpy(self):
        """K as [page][H][D / 16][PT][16] and V^T as [page][H][D][PT], uint16 bit patterns (V^T is stored in runs of
        min(PT, 32) keys, [page][H][PT / run][D][run]; the runs are put back side by side here)."""
        import numpy as np
        g = self.geom
        k = self.k.cpu().numpy().view(np.uint16).reshape(g.n_pages, g.n_kv_heads, g.head_dim // 16, g.page_tokens, 16)
        run = min(g.page_tokens, 32)
        v = self.v.cpu().numpy().view(np.uint16).reshape(g.n_pages, g.n_kv_heads, g.page_tokens // run, g.head_dim, run)
        v = v.transpose(0, 1, 3, 2, 4).reshape(g.n_pages, g.n_kv_heads, g.head_dim, g.page_tokens)
        return k, v


def f16_geometry(n_q_heads, n_kv_heads, head_dim, page_tokens, n_pages):
    g = geometry(Q8_0, n_q_heads, n_kv_heads, head_dim, page_tokens, n_pages)  # the same limits
    g.format = KV_F16
    return g


def f16_append(pools, table, start_pos, k_src, v_src, n_valid=None):
    """append() for f16 pools: rows rounded to f16 and written at their page rows."""
    g = pools.geom
    assert k_src.is_contiguous() and v_src.is_contiguous() and table.is_contiguous() and k_src.dtype == v_src.dtype
    n_seqs, n_new = k_src.shape[0], k_src.shape[1]
    assert tuple(k_src.shape) == (n_seqs, n_new, g.n_kv_heads, g.head_dim) and k_src.shape == v_src.shape
    st = pools.struct()
    _check(lib.yahkv_f16_append(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(start_pos), _dp(n_valid),
                                n_seqs, n_new, _dp(k_src), _dp(v_src), _dtype_code(k_src), _stream()), "f16_append")


def f16_decode_attend(pools, table, seq_len, max_seq_len, q, scale, gate=None, out=None, workspace=None, opt=None):
    """decode_attend() over f16 pools; returns out f32 [n_seqs][n_q_heads][D]."""
    import torch
    g = pools.geom
    n_seqs = q.shape[0]
    assert q.is_contiguous() and table.is_contiguous() and tuple(q.shape) == (n_seqs, g.n_q_heads, g.head_dim)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    if workspace is None:
        need = lib.yahkv_f16_decode_workspace_bytes(C.byref(g), n_seqs, max_seq_len, _op(opt))
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    st = pools.struct()
    _check(lib.yahkv_f16_decode_attend(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), n_seqs,
                                       max_seq_len, _dp(q), _dtype_code(q), scale, _dp(gate), _dp(out),
                                       _dp(workspace), workspace.numel(), _op(opt), _stream()), "f16_decode_attend")
    return out


def f16_prefill_attend(pools, table, prefix_len, max_prefix_len, q, scale, gate=None, out=None, workspace=None):
    """prefill_attend() over f16 pools; q bf16 [n_seqs][chunk][n_q_heads][D]; returns out (f16 unless given)."""
    import torch
    g = pools.geom
    n_seqs, chunk = q.shape[0], q.shape[1]
    assert q.is_contiguous() and q.dtype == torch.bfloat16 and tuple(q.shape[2:]) == (g.n_q_heads, g.head_dim)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    if workspace is None:
        need = lib.yahkv_f16_prefill_workspace_bytes(C.byref(g), n_seqs, max_prefix_len, chunk)
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    st = pools.struct()
    _check(lib.yahkv_f16_prefill_attend(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(prefix_len), n_seqs,
                                        max_prefix_len, chunk, _dp(q), scale, _dp(gate), _dp(out), _dtype_code(out),
                                        _dp(workspace), workspace.numel(), _stream()), "f16_prefill_attend")
    return out


class DevicePools:
    """One layer's four pools on the GPU (LoomDecoderState's kq / ks / vq / vs)."""

    def __init__(self, g, fill=0, device="cuda:0"):
        import torch
        self.geom = g
        b = pool_bytes(g)
        self.kq = torch.full((b["kq"],), fill, dtype=torch.uint8, device=device)
        self.ks = torch.full((b["ks"],), fill, dtype=torch.uint8, device=device)
        self.vq = torch.full((b["vq"],), fill, dtype=torch.uint8, device=device)
        self.vs = torch.full((b["vs"],), fill, dtype=torch.uint8, device=device)

    def struct(self):
        return Pools(self.kq.data_ptr(), self.ks.data_ptr(), self.vq.data_ptr(), self.vs.data_ptr(),
                     self.kq.numel(), self.ks.numel(), self.vq.numel(), self.vs.numel())

    def numpy(self):
        import numpy as np
        return {"kq": self.kq.cpu().numpy(), "ks": self.ks.cpu().numpy().view(np.uint16),
                "vq": self.vq.cpu().numpy(), "vs": self.vs.cpu().numpy().view(np.uint16)}

    def load(self, arrays):
        """Upload host pools (numpy arrays keyed kq / ks / vq / vs)."""
        import numpy as np
        import torch
        for name in ("kq", "ks", "vq", "vs"):
            src = torch.from_numpy(np.ascontiguousarray(arrays[name]).view(np.uint8).reshape(-1))
            getattr(self, name).copy_(src)


def append(pools, table, start_pos, k_src, v_src, n_valid=None):
    """k_src / v_src: [n_seqs][n_new][H][D] f32 / f16 / bf16 cuda tensors; table int32 [n_seqs][stride]."""
    g = pools.geom
    assert k_src.is_contiguous() and v_src.is_contiguous() and table.is_contiguous() and k_src.dtype == v_src.dtype
    n_seqs, n_new = k_src.shape[0], k_src.shape[1]
    assert tuple(k_src.shape) == (n_seqs, n_new, g.n_kv_heads, g.head_dim) and k_src.shape == v_src.shape
    st = pools.struct()
    _check(lib.yahkv_append(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(start_pos), _dp(n_valid),
                            n_seqs, n_new, _dp(k_src), _dp(v_src), _dtype_code(k_src), _stream()), "append")


def append_rope(pools, table, start_pos, k_src, v_src, theta, eps, rotary_dim, k_weight=None, q_weight=None, q_src=None,
                q_out_dtype=None, want_k=False, n_valid=None):
    """append() with per-head RMSNorm + NeoX RoPE of K fused in (position of token t of sequence s: start_pos[s] + t).
    q_src [n_seqs][n_new][n_q_heads][D] is normalised and rotated into the returned q_out; want_k also returns the
    rotated K rows as f32. Returns (q_out or None, k_out or None)."""
    import torch
    g = pools.geom
    assert k_src.is_contiguous() and v_src.is_contiguous() and table.is_contiguous() and k_src.dtype == v_src.dtype
    n_seqs, n_new = k_src.shape[0], k_src.shape[1]
    assert tuple(k_src.shape) == (n_seqs, n_new, g.n_kv_heads, g.head_dim) and k_src.shape == v_src.shape
    q_out = None
    if q_src is not None:
        assert q_src.is_contiguous() and q_src.dtype == k_src.dtype
        assert tuple(q_src.shape) == (n_seqs, n_new, g.n_q_heads, g.head_dim)
        q_out = torch.empty(q_src.shape, dtype=q_out_dtype or torch.float32, device=q_src.device)
    k_out = torch.empty(k_src.shape, dtype=torch.float32, device=k_src.device) if want_k else None
    rope = Rope(theta, eps, rotary_dim, _dp(k_weight), _dp(q_weight))
    st = pools.struct()
    _check(lib.yahkv_append_rope(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(start_pos), _dp(n_valid),
                                 n_seqs, n_new, _dp(k_src), _dp(v_src), _dtype_code(k_src), C.byref(rope), _dp(q_src),
                                 _dp(q_out), _dtype_code(q_out) if q_out is not None else 0, _dp(k_out), _stream()),
           "append_rope")
    return q_out, k_out


def decode_options(n_chunks=0, min_chunk_tiles=0, pair_cost=0, reduce_split=0, deterministic=False, xcd_weight=None,
                   one_launch=False, wg_partials=0, cut=0):
    """yahkv_decode_options; zero / None fields are the defaults."""
    o = DecodeOptions(n_chunks, min_chunk_tiles, pair_cost, reduce_split, 1 if deterministic else 0)
    o.one_launch = 1 if one_launch else 0
    o.wg_partials = int(wg_partials)
    o.cut = int(cut)
    for j, w in enumerate(xcd_weight or ()):
        o.xcd_weight[j] = int(w)
    return o


def _op(opt):
    return None if opt is None else C.byref(opt)


def decode_workspace_bytes(g, n_seqs, max_seq_len, opt=None):
    return lib.yahkv_decode_workspace_bytes(C.byref(g), n_seqs, max_seq_len, _op(opt))


def decode_workspace_init(g, n_seqs, max_seq_len, workspace, opt=None):
    """Zeroes the arrival counts the one-launch form keeps in the workspace (once per workspace and shape)."""
    _check(lib.yahkv_decode_workspace_init(C.byref(g), n_seqs, max_seq_len, _op(opt), _dp(workspace), workspace.numel(),
                                           _stream()), "decode_workspace_init")


def decode_attend(pools, table, seq_len, max_seq_len, q, scale, gate=None, out=None, workspace=None, opt=None):
    """q: [n_seqs][n_q_heads][D] f16 / bf16 / f32; returns out f32 of the same shape. A workspace given by the caller
    and used with opt.one_launch must have been through decode_workspace_init."""
    import torch
    g = pools.geom
    n_seqs = q.shape[0]
    assert q.is_contiguous() and table.is_contiguous() and tuple(q.shape) == (n_seqs, g.n_q_heads, g.head_dim)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    need = decode_workspace_bytes(g, n_seqs, max_seq_len, opt)
    if workspace is None:
        workspace = torch.empty(need, dtype=torch.uint8, device=q.device)
        if opt is not None and opt.one_launch:
            decode_workspace_init(g, n_seqs, max_seq_len, workspace, opt)
    st = pools.struct()
    _check(lib.yahkv_decode_attend(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), n_seqs,
                                   max_seq_len, _dp(q), _dtype_code(q), scale, _dp(gate), _dp(out), _dp(workspace),
                                   workspace.numel(), _op(opt), _stream()), "decode_attend")
    return out


def decode_step(pools, table, seq_len, max_seq_len, k_new, v_new, q, scale, gate=None, out=None, workspace=None,
                opt=None):
    """Append + attention of one decode step in two dispatches. seq_len counts the step's own token, whose K / V rows
    are k_new, v_new [n_seqs][n_kv_heads][D] (f32 / f16 / bf16); q as for decode_attend. Returns out f32."""
    import torch
    g = pools.geom
    n_seqs = q.shape[0]
    assert q.is_contiguous() and table.is_contiguous() and tuple(q.shape) == (n_seqs, g.n_q_heads, g.head_dim)
    assert k_new.is_contiguous() and v_new.is_contiguous() and k_new.dtype == v_new.dtype
    assert tuple(k_new.shape) == tuple(v_new.shape) == (n_seqs, g.n_kv_heads, g.head_dim)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    if workspace is None:
        workspace = torch.empty(decode_workspace_bytes(g, n_seqs, max_seq_len, opt), dtype=torch.uint8, device=q.device)
    st = pools.struct()
    _check(lib.yahkv_decode_step(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), n_seqs, max_seq_len,
                                 _dp(k_new), _dp(v_new), _dtype_code(k_new), _dp(q), _dtype_code(q), scale, _dp(gate),
                                 _dp(out), _dp(workspace), workspace.numel(), _op(opt), _stream()), "decode_step")
    return out


def decode_step_reduce(pools, table, seq_len, max_seq_len, k_new, v_new, q, scale, out, workspace, gate=None, opt=None):
    """Second dispatch of decode_step (the first: decode_part on the lengths before the step)."""
    g = pools.geom
    st = pools.struct()
    _check(lib.yahkv_decode_step_reduce(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                        max_seq_len, _dp(k_new), _dp(v_new), _dtype_code(k_new), _dp(q), _dtype_code(q),
                                        scale, _dp(gate), _dp(out), _dp(workspace), workspace.numel(), _op(opt),
                                        _stream()), "decode_step_reduce")
    return out


def shader_clock_probe(out, ticks=2000):
    """Queues the clock probe; out: an int64 cuda tensor of two elements, {shader cycles, 100 MHz ticks} once it ran."""
    _check(lib.yahkv_shader_clock_probe(_dp(out), ticks, _stream()), "shader_clock_probe")


def decode_attend_static(pools, table, seq_len, max_seq_len, q, scale, out, gate=None):
    """decode_attend() on the library's own scratch array: no workspace, no allocation (out is the caller's)."""
    g = pools.geom
    st = pools.struct()
    _check(lib.yahkv_decode_attend_static(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                          max_seq_len, _dp(q), _dtype_code(q), scale, _dp(gate), _dp(out), _stream()),
           "decode_attend_static")
    return out


def decode_part(pools, table, seq_len, max_seq_len, q, scale, workspace, opt=None):
    """First dispatch of decode_attend: partials into the workspace."""
    g = pools.geom
    st = pools.struct()
    _check(lib.yahkv_decode_part(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                 max_seq_len, _dp(q), _dtype_code(q), scale, _dp(workspace), workspace.numel(),
                                 _op(opt), _stream()), "decode_part")


def decode_step_calls(pools, table, seq_len_before, seq_len, max_seq_len, k_new, v_new, q, scale, out, workspace,
                      gate=None, opt=None):
    """The two calls of one decode step (decode_part on the lengths before the step, decode_step_reduce on the lengths
    with it) with their arguments marshalled once: returns (part, reduce), two functions of no arguments. A loop that
    issues many steps (a benchmark, a server) then pays for the two C calls alone, as a C++ caller does, and not for
    building ctypes arguments from tensors on every step. The tensors must stay alive and in place; the stream is the
    one current now unless a call names another."""
    g = pools.geom
    st = pools.struct()
    stream = _stream()
    common = (C.byref(g), C.byref(st), _dp(table), table.shape[1])
    part_args = common + (_dp(seq_len_before), q.shape[0], max_seq_len, _dp(q), _dtype_code(q), scale, _dp(workspace),
                          workspace.numel(), _op(opt))
    reduce_args = common + (_dp(seq_len), q.shape[0], max_seq_len, _dp(k_new), _dp(v_new), _dtype_code(k_new), _dp(q),
                            _dtype_code(q), scale, _dp(gate), _dp(out), _dp(workspace), workspace.numel(), _op(opt))
    keep = (g, st, table, seq_len_before, seq_len, k_new, v_new, q, out, workspace, gate, opt)
    fp, fr = lib.yahkv_decode_part, lib.yahkv_decode_step_reduce

    def part(on=stream, _keep=keep):  # on: another stream's handle (a ctypes void pointer), e.g. one that is being captured
        rc = fp(*part_args, on)
        if rc:
            _check(rc, "decode_part")

    def reduce(on=stream, _keep=keep):
        rc = fr(*reduce_args, on)
        if rc:
            _check(rc, "decode_step_reduce")

    return part, reduce


def decode_reduce(g, table_stride, seq_len, n_seqs, max_seq_len, out, workspace, gate=None, opt=None):
    """Second dispatch of decode_attend: merge the partials into out."""
    _check(lib.yahkv_decode_reduce(C.byref(g), table_stride, _dp(seq_len), n_seqs, max_seq_len, _dp(gate), _dp(out),
                                   _dp(workspace), workspace.numel(), _op(opt), _stream()), "decode_reduce")


def decode_calibrate(pools, table, seq_len, max_seq_len, q, workspace, opt, rounds=2):
    """Measures the XCDs' relative speeds on this batch into opt.xcd_weight (synchronizes; overwrites the workspace)."""
    g = pools.geom
    st = pools.struct()
    _check(lib.yahkv_decode_calibrate(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                      max_seq_len, _dp(q), _dtype_code(q), _dp(workspace), workspace.numel(),
                                      C.byref(opt), rounds, _stream()), "decode_calibrate")
    return list(opt.xcd_weight)


def prefill_workspace_bytes(g, n_seqs, max_prefix_len, chunk_len):
    return lib.yahkv_prefill_workspace_bytes(C.byref(g), n_seqs, max_prefix_len, chunk_len)


def prefill_attend(pools, table, prefix_len, max_prefix_len, q, scale, gate=None, out=None, out_dtype=None,
                   workspace=None):
    """q: [n_seqs][chunk][n_q_heads][D] bf16; returns out (f32 unless out / out_dtype say otherwise), same shape.

    workspace: a uint8 device tensor of prefill_workspace_bytes() (None: one is allocated for the call) selects the
    two-pass path, decode to f16 tile images and then attention; False selects the one-pass kernel."""
    import torch
    g = pools.geom
    assert q.is_contiguous() and q.dtype == torch.bfloat16 and table.is_contiguous()
    if out is None:
        out = torch.empty(q.shape, dtype=out_dtype or torch.float32, device=q.device)
    if workspace is None:
        workspace = torch.empty(prefill_workspace_bytes(g, q.shape[0], max_prefix_len, q.shape[1]), dtype=torch.uint8,
                                device=q.device)
    ws_ptr, ws_bytes = (None, 0) if workspace is False else (_dp(workspace), workspace.numel())
    st = pools.struct()
    _check(lib.yahkv_prefill_attend(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(prefix_len), q.shape[0],
                                    max_prefix_len, q.shape[1], _dp(q), scale, _dp(gate), _dp(out), _dtype_code(out),
                                    ws_ptr, ws_bytes, _stream()), "prefill_attend")
    return out


def prefill_decode_tiles(pools, table, prefix_len, max_prefix_len, n_seqs, chunk_len, workspace):
    """First dispatch of the workspace path of prefill_attend: K / V of prefix + chunk as bf16 tiles in workspace."""
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_prefill_decode_tiles(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(prefix_len), n_seqs,
                                          max_prefix_len, chunk_len, _dp(workspace), workspace.numel(), _stream()),
           "prefill_decode_tiles")


def prefill_attend_tiles(pools, table, prefix_len, max_prefix_len, q, scale, out, workspace, gate=None):
    """Second dispatch: attention of the chunk's queries over the tiles in workspace."""
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_prefill_attend_tiles(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(prefix_len),
                                          q.shape[0], max_prefix_len, q.shape[1], _dp(q), scale, _dp(gate), _dp(out),
                                          _dtype_code(out), _dp(workspace), workspace.numel(), _stream()),
           "prefill_attend_tiles")
    return out


def copy_pages(pools, src_pages, dst_pages):
    """Whole pages src_pages[i] -> dst_pages[i] (int32 cuda tensors) in all four pools."""
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_copy_pages(C.byref(g), C.byref(st), _dp(src_pages), _dp(dst_pages), src_pages.numel(), _stream()),
           "copy_pages")


def slot_pack(pools, table_row, n_pages, n_tokens):
    """The first n_pages pages of a sequence (table_row: int32 cuda tensor) as one uint8 cuda tensor: header + pages."""
    import torch
    g, st = pools.geom, pools.struct()
    slot = torch.empty(lib.yahkv_slot_bytes(C.byref(g), n_pages), dtype=torch.uint8, device=table_row.device)
    _check(lib.yahkv_slot_pack(C.byref(g), C.byref(st), _dp(table_row), n_pages, n_tokens, _dp(slot), _stream()),
           "slot_pack")
    return slot


def slot_check(g, slot_host):
    """slot_host: numpy uint8 array of a whole slot; returns (n_pages, n_tokens) or raises."""
    n_pages, n_tokens = C.c_int32(), C.c_int32()
    _check(lib.yahkv_slot_check(C.byref(g), slot_host.ctypes.data, slot_host.nbytes, C.byref(n_pages),
                                C.byref(n_tokens)), "slot_check")
    return n_pages.value, n_tokens.value


def slot_unpack(pools, table_row, n_pages, slot):
    """Scatter a slot (uint8 cuda tensor) into the pages named by table_row[:n_pages]."""
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_slot_unpack(C.byref(g), C.byref(st), _dp(table_row), n_pages, _dp(slot), _stream()), "slot_unpack")


def gather_blocks(pools, table_row, n_tokens):
    """Blocks of tokens [0, n_tokens) of one sequence in ggml order: two uint8 tensors [n][H][NB][34 | 18]."""
    import torch
    g = pools.geom
    bb = 34 if g.format == Q8_0 else 18
    shape = (n_tokens, g.n_kv_heads, g.head_dim // 32, bb)
    k = torch.zeros(shape, dtype=torch.uint8, device=table_row.device)
    v = torch.zeros(shape, dtype=torch.uint8, device=table_row.device)
    st = pools.struct()
    _check(lib.yahkv_gather_blocks(C.byref(g), C.byref(st), _dp(table_row), n_tokens, _dp(k), _dp(v), _stream()),
           "gather_blocks")
    return k, v


# ---- kv8a16: the reference's own KV format (yahkv_kv8_*) --------------------------------------------------------------

def kv8_geometry(n_q_heads, n_kv_heads, n_pages, k_bits=8, v_bits=8):
    """The reference's own formats: kv8a16 (8, 8), kv4a16 (4, 4) and the mixes k8v4 / k4v8."""
    g = Geometry(_KV8_FORMATS[(k_bits, v_bits)], n_q_heads, n_kv_heads, 256, 256, n_pages)
    if lib.yahkv_kv8_kq_bytes(C.byref(g)) == 0:
        raise YahkvError(-2, "kv8a16 / kv4a16 geometry")
    return g


class Kv8Pools:
    """One layer's kv8a16 buffers on the GPU, in the reference's layouts: kq, ks, vq, vs (LoomDecoderState), and per page
    the channel means (km) and the open V tile (vopen)."""

    NAMES = Kv8PoolsStruct._NAMES

    def __init__(self, g, fill=0, device="cuda:0"):
        import torch
        assert g.format in _KV8_FORMATS.values()
        self.geom = g
        self.k_bits, self.v_bits = next(kv for kv, f in _KV8_FORMATS.items() if f == g.format)
        for n in self.NAMES:
            nbytes = getattr(lib, f"yahkv_kv8_{n}_bytes")(C.byref(g))
            setattr(self, n, torch.full((nbytes,), fill, dtype=torch.uint8, device=device))

    def struct(self):
        return Kv8PoolsStruct(*[getattr(self, n).data_ptr() for n in self.NAMES],
                              *[getattr(self, n).numel() for n in self.NAMES])

    def numpy(self):
        """The buffers as the arrays documented in include/yahkv.h (vopen under the oracle's name `vo`)."""
        import numpy as np
        g = self.geom
        H, P, W = g.n_kv_heads, g.n_pages, g.n_kv_heads * 256
        raw = {n: getattr(self, n).cpu().numpy() for n in self.NAMES}
        kqw, ksw, vqw = (W // 8, W // 32) if self.k_bits == 4 else (W // 4, W // 128), None, 2 if self.v_bits == 4 else 4
        kqw, ksw = kqw
        return {"kq": raw["kq"].view(np.uint32).reshape(P * 256, kqw), "ks": raw["ks"].view(np.uint32).reshape(P * 256, ksw),
                "km": raw["km"].view(np.float32).reshape(P, W), "vq": raw["vq"].view(np.uint32).reshape(H, P * 16, 256, vqw),
                "vs": raw["vs"].view(np.uint32).reshape(H, P * 16, 256), "vo": raw["vopen"].view(np.uint16).reshape(P, W, 16)}

    def load(self, arrays):
        import numpy as np
        import torch
        for n in self.NAMES:
            a = arrays["vo" if n == "vopen" else n]
            getattr(self, n).copy_(torch.from_numpy(np.ascontiguousarray(a).view(np.uint8).reshape(-1)))


def kv8_copy_pages(pools, src_pages, dst_pages):
    """Whole pages src_pages[i] -> dst_pages[i] (int32 cuda tensors) in all six buffers."""
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_kv8_copy_pages(C.byref(g), C.byref(st), _dp(src_pages), _dp(dst_pages), src_pages.numel(), _stream()),
           "kv8_copy_pages")


def kv8_slot_pack(pools, table_row, n_pages, n_tokens):
    """The sequence's pages (device int32 row) as one uint8 cuda tensor: header + pools of n_pages pages, identity table."""
    import torch
    g, st = pools.geom, pools.struct()
    slot = torch.empty(lib.yahkv_kv8_slot_bytes(C.byref(g), n_pages), dtype=torch.uint8, device=table_row.device)
    _check(lib.yahkv_kv8_slot_pack(C.byref(g), C.byref(st), _dp(table_row), n_pages, n_tokens, _dp(slot), _stream()),
           "kv8_slot_pack")
    return slot


def kv8_slot_check(g, slot_host):
    """(n_pages, n_tokens) of a slot held in a uint8 numpy array; raises where the geometry does not match."""
    np_, nt = C.c_int32(0), C.c_int32(0)
    _check(lib.yahkv_kv8_slot_check(C.byref(g), C.c_void_p(slot_host.ctypes.data), C.c_size_t(slot_host.size), C.byref(np_),
                                    C.byref(nt)), "kv8_slot_check")
    return np_.value, nt.value


def kv8_slot_unpack(pools, table_row, n_pages, slot):
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_kv8_slot_unpack(C.byref(g), C.byref(st), _dp(table_row), n_pages, _dp(slot), _stream()), "kv8_slot_unpack")


class RefSlotInfo(C.Structure):
    _fields_ = [("context", C.c_uint64), ("chunk", C.c_uint64), ("chunks", C.c_uint64), ("n_pages", C.c_int32),
                ("n_layers", C.c_int32), ("n_kv_heads", C.c_int32), ("format", C.c_int32), ("offset", C.c_uint64 * 10),
                ("size", C.c_uint64 * 10)]


def refslot_parse(file_bytes):
    """Validates a slot file of the reference ("YAHSLOT1", loom_prefill.hpp:976-1024) held in a bytes-like object or a
    uint8 numpy array and says what it holds. Host only."""
    import numpy as np
    buf = np.frombuffer(file_bytes, np.uint8) if not isinstance(file_bytes, np.ndarray) else file_bytes
    info = RefSlotInfo()
    _check(lib.yahkv_refslot_parse(C.c_void_p(buf.ctypes.data), C.c_size_t(buf.size), C.byref(info)), "refslot_parse")
    return info


def refslot_load_layer(pools, file_bytes, layer, pages):
    """One layer's pages of a reference slot file into pages[...] (logical order) of kv8a16 / kv4a16 pools."""
    import numpy as np
    buf = np.frombuffer(file_bytes, np.uint8) if not isinstance(file_bytes, np.ndarray) else file_bytes
    pg = np.ascontiguousarray(pages, np.int32)
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_refslot_load_layer(C.byref(g), C.byref(st), C.c_void_p(buf.ctypes.data), C.c_size_t(buf.size),
                                        int(layer), C.c_void_p(pg.ctypes.data), int(pg.size), _stream()), "refslot_load_layer")


def kv8_kmean(pools, table, k_src, n_valid=None):
    """Channel means of each sequence's first chunk k_src [n_seqs][n_rows][H][256], written to km of its first page."""
    g = pools.geom
    assert k_src.is_contiguous() and table.is_contiguous() and tuple(k_src.shape[2:]) == (g.n_kv_heads, 256)
    st = pools.struct()
    _check(lib.yahkv_kv8_kmean(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(n_valid), k_src.shape[0],
                               k_src.shape[1], _dp(k_src), _dtype_code(k_src), _stream()), "kv8_kmean")


def kv8_append(pools, table, start_pos, k_src, v_src, n_valid=None):
    """k_src / v_src: [n_seqs][n_new][H][256]; n_new == 1 is the decoder's append, more the prefill's chunk."""
    g = pools.geom
    assert k_src.is_contiguous() and v_src.is_contiguous() and table.is_contiguous() and k_src.dtype == v_src.dtype
    assert tuple(k_src.shape[2:]) == (g.n_kv_heads, 256) and k_src.shape == v_src.shape
    st = pools.struct()
    _check(lib.yahkv_kv8_append(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(start_pos), _dp(n_valid),
                                k_src.shape[0], k_src.shape[1], _dp(k_src), _dp(v_src), _dtype_code(k_src), _stream()),
           "kv8_append")


def _kv8_out_ws(g, q, n_seqs, max_seq_len, out, workspace, opt):
    import torch
    assert q.is_contiguous() and tuple(q.shape) == (n_seqs, g.n_q_heads, 256)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    if workspace is None:
        need = lib.yahkv_kv8_decode_workspace_bytes(C.byref(g), n_seqs, max_seq_len, _op(opt))
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    return out, workspace


def kv8_decode_attend(pools, table, seq_len, max_seq_len, q, scale, gate=None, out=None, workspace=None, opt=None):
    g = pools.geom
    out, workspace = _kv8_out_ws(g, q, q.shape[0], max_seq_len, out, workspace, opt)
    st = pools.struct()
    _check(lib.yahkv_kv8_decode_attend(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                       max_seq_len, _dp(q), _dtype_code(q), scale, _dp(gate), _dp(out), _dp(workspace),
                                       workspace.numel(), _op(opt), _stream()), "kv8_decode_attend")
    return out


def kv8_decode_step(pools, table, seq_len, max_seq_len, k_new, v_new, q, scale, gate=None, out=None, workspace=None,
                    opt=None):
    """seq_len counts the step's token; k_new / v_new [n_seqs][H][256]."""
    g = pools.geom
    assert k_new.is_contiguous() and v_new.is_contiguous() and k_new.dtype == v_new.dtype
    out, workspace = _kv8_out_ws(g, q, q.shape[0], max_seq_len, out, workspace, opt)
    st = pools.struct()
    _check(lib.yahkv_kv8_decode_step(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                     max_seq_len, _dp(k_new), _dp(v_new), _dtype_code(k_new), _dp(q), _dtype_code(q),
                                     scale, _dp(gate), _dp(out), _dp(workspace), workspace.numel(), _op(opt), _stream()),
           "kv8_decode_step")
    return out


def kv8_prefill_attend(pools, table, prefix_len, max_prefix_len, q, scale, gate=None, out=None, workspace=None):
    """prefill_attend() over kv8a16 pools; q bf16 [n_seqs][chunk][n_q_heads][256]; returns out (f16 unless given)."""
    import torch
    g = pools.geom
    n_seqs, chunk = q.shape[0], q.shape[1]
    assert q.is_contiguous() and q.dtype == torch.bfloat16 and tuple(q.shape[2:]) == (g.n_q_heads, 256)
    if out is None:
        out = torch.empty(q.shape, dtype=torch.float16, device=q.device)
    if workspace is None:
        need = lib.yahkv_kv8_prefill_workspace_bytes(C.byref(g), n_seqs, max_prefix_len, chunk)
        workspace = torch.empty(max(need, 16), dtype=torch.uint8, device=q.device)
    st = pools.struct()
    _check(lib.yahkv_kv8_prefill_attend(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(prefix_len), n_seqs,
                                        max_prefix_len, chunk, _dp(q), scale, _dp(gate), _dp(out), _dtype_code(out),
                                        _dp(workspace), workspace.numel(), _stream()), "kv8_prefill_attend")
    return out


def kv8_decode_calibrate(pools, table, seq_len, max_seq_len, q, workspace, opt, rounds=2):
    """Measures the XCDs' relative read speeds on this batch into opt.xcd_weight; returns them as a list."""
    g, st = pools.geom, pools.struct()
    _check(lib.yahkv_kv8_decode_calibrate(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                          max_seq_len, _dp(q), _dtype_code(q), _dp(workspace), C.c_size_t(workspace.numel()),
                                          C.byref(opt), int(rounds), _stream()), "kv8_decode_calibrate")
    return list(opt.xcd_weight)


def kv8_decode_part(pools, table, seq_len, max_seq_len, q, scale, workspace, opt=None):
    g = pools.geom
    st = pools.struct()
    _check(lib.yahkv_kv8_decode_part(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                     max_seq_len, _dp(q), _dtype_code(q), scale, _dp(workspace), workspace.numel(),
                                     _op(opt), _stream()), "kv8_decode_part")


def kv8_decode_reduce(pools, table, seq_len, max_seq_len, q, scale, out, workspace, k_new=None, v_new=None, gate=None,
                      opt=None):
    """The merge; with k_new / v_new [n_seqs][H][256] the step's (it appends that token and attends to it)."""
    g = pools.geom
    st = pools.struct()
    _check(lib.yahkv_kv8_decode_reduce(C.byref(g), C.byref(st), _dp(table), table.shape[1], _dp(seq_len), q.shape[0],
                                       max_seq_len, _dp(k_new), _dp(v_new), 0 if k_new is None else _dtype_code(k_new),
                                       _dp(q), _dtype_code(q), scale, _dp(gate), _dp(out), _dp(workspace),
                                       workspace.numel(), _op(opt), _stream()), "kv8_decode_reduce")
