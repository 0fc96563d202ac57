"""The inputs of the reference's kv8a16 checker (engine/gpu/loom/tools/dattn_q_check.py:140-256: rng 5, T 1024,
pos 700, a scrambled page table), drawn again from its seed in its order, for the CPU and GPU tests of the kv8a16
format. The expected outputs come from tests/golden/kv8a16_vectors.npz, which also holds digests of the inputs drawn
here: if numpy ever changes the stream of default_rng(5), load() says so instead of comparing against other data."""
import hashlib
import os

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
f32, f16 = np.float32, np.float16


def sha(a):
    return np.frombuffer(hashlib.sha256(np.ascontiguousarray(a).tobytes()).digest(), np.uint8)


def golden(bits=8):
    return np.load(os.path.join(ROOT, "tests", "golden", "kv%da16_vectors.npz" % bits), allow_pickle=False)


class Recipe:
    pass


def load(bits=8):
    """bits = 4: the same draws (the checker's stream does not depend on the format) with kv4a16_vectors.npz's outputs"""
    g = golden(bits)
    r = Recipe()
    r.bits = bits
    r.g = g
    r.T, r.pos = int(g["rc_T"]), int(g["rc_pos"])
    rng = np.random.default_rng(5)
    r.ptab = rng.permutation(r.T // 256).astype(np.int32)
    r.m = (0.5 * rng.standard_normal(1024)).astype(f32)
    r.K = (rng.standard_normal((r.T, 1024)) + r.m).astype(f16)
    r.V = rng.standard_normal((r.T, 1024)).astype(f16)
    r.q = (0.3 * rng.standard_normal((24, 256))).astype(f32)
    r.gate = rng.standard_normal((24, 256)).astype(f32)
    for name, mine in (("rc_ptab", r.ptab), ("rc_m", r.m), ("rc_q", r.q), ("rc_gate", r.gate)):
        assert np.array_equal(g[name], mine), f"default_rng(5) no longer draws the fixture's {name}"
    assert np.array_equal(g["rc_K_sha"], sha(r.K)) and np.array_equal(g["rc_V_sha"], sha(r.V)), \
        "default_rng(5) no longer draws the fixture's K / V"
    r.n = r.pos + 1
    r.curt = r.pos // 16
    r.nk = r.pos - 16 * r.curt + 1
    return r


def prow(r, p):
    return int(r.ptab[p // 256]) * 256 + p % 256


def ptile(r, t):
    return int(r.ptab[t // 16]) * 16 + t % 16
