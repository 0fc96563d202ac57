"""The oracle's RMSNorm + NeoX RoPE (orc_norm_rope, after engine/gpu/loom/yah_fused_qk_rope_f32.loom:96-146). The
reference holds no vectors for that kernel, so the restatement is pinned by what the mathematics fixes: a
hand-computed answer, the identity at position 0, rotations preserving pair norms, the relative-position property,
and an independent float64 form."""
import numpy as np

import oracle


def numpy_norm_rope(x, w, rot, theta, eps, pos):
    x = x.astype(np.float64)
    d = x.shape[-1]
    n = x / np.sqrt((x * x).mean(-1, keepdims=True) + eps) * (1.0 if w is None else w.astype(np.float64))
    half = rot // 2
    ang = np.asarray(pos, np.float64)[..., None] / theta ** (2.0 * np.arange(half) / rot)
    out = n.copy()
    out[..., :half] = n[..., :half] * np.cos(ang) - n[..., half:rot] * np.sin(ang)
    out[..., half:rot] = n[..., :half] * np.sin(ang) + n[..., half:rot] * np.cos(ang)
    return out


def test_known_answer_half_split_pairs():
    # D = rotary_dim = 4: pairs are (0, 2) and (1, 3); x = e0 has rms 1/2, so normed = 2 e0; at pos 1 the pair (0, 2)
    # turns by 1 rad (p = 0: theta^0 = 1). An interleaved pairing would put the sine into element 1 instead.
    out = oracle.norm_rope(np.array([[1.0, 0, 0, 0]], np.float32), None, 4, 10000.0, 0.0, [1])
    assert np.allclose(out, [[2 * np.cos(1.0), 0, 2 * np.sin(1.0), 0]], atol=1e-6)
    # e1 turns by pos / theta^(2/4) = 3 / 100
    out = oracle.norm_rope(np.array([[0, 1.0, 0, 0]], np.float32), None, 4, 10000.0, 0.0, [3])
    assert np.allclose(out, [[0, 2 * np.cos(0.03), 0, 2 * np.sin(0.03)]], atol=1e-6)
    # weights scale after the normalisation, before the rotation; eps enters under the root
    out = oracle.norm_rope(np.array([[3.0, 0, 0, 0]], np.float32), np.array([0.5, 1, 1, 1], np.float32), 4, 10000.0, 0.75, [0])
    assert np.allclose(out, [[3 / np.sqrt(9 / 4 + 0.75) * 0.5, 0, 0, 0]], atol=1e-6)


def test_position_zero_is_the_norm_and_tail_dims_are_not_rotated():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((5, 128)).astype(np.float32)
    w = rng.standard_normal(128).astype(np.float32)
    at0 = oracle.norm_rope(x, w, 64, 1e6, 1e-6, [0] * 5)
    want = x / np.sqrt((x.astype(np.float64) ** 2).mean(-1, keepdims=True) + 1e-6) * w
    assert np.allclose(at0, want, rtol=1e-5, atol=1e-6)
    far = oracle.norm_rope(x, w, 64, 1e6, 1e-6, [977] * 5)
    assert np.array_equal(far[:, 64:], at0[:, 64:])          # dims at or past rotary_dim
    assert not np.allclose(far[:, :64], at0[:, :64], atol=1e-3)
    # a rotation keeps the norm of every pair (p, p + 32)
    assert np.allclose(far[:, :32] ** 2 + far[:, 32:64] ** 2, at0[:, :32] ** 2 + at0[:, 32:64] ** 2, rtol=1e-4, atol=1e-6)


def test_dot_products_depend_on_the_position_difference_only():
    rng = np.random.default_rng(1)
    q = rng.standard_normal((1, 256)).astype(np.float32)
    k = rng.standard_normal((1, 256)).astype(np.float32)
    dots = []
    for m, n in ((10, 3), (107, 100), (1007, 1000)):
        a = oracle.norm_rope(q, None, 256, 1e7, 1e-6, [m]).astype(np.float64)
        b = oracle.norm_rope(k, None, 256, 1e7, 1e-6, [n]).astype(np.float64)
        dots.append(float((a * b).sum()))
    assert abs(dots[0] - dots[1]) < 2e-3 * 256 and abs(dots[0] - dots[2]) < 2e-3 * 256   # f32 angles at pos 1000
    a = oracle.norm_rope(q, None, 256, 1e7, 1e-6, [10]).astype(np.float64)
    b = oracle.norm_rope(k, None, 256, 1e7, 1e-6, [4]).astype(np.float64)
    assert abs(float((a * b).sum()) - dots[0]) > 1e-2                                     # another difference differs


def test_against_float64_form():
    rng = np.random.default_rng(2)
    for d, rot, theta in ((128, 128, 1e4), (256, 256, 1e7), (256, 64, 1e6)):
        x = rng.standard_normal((7, 3, d)).astype(np.float32)
        w = (1 + 0.1 * rng.standard_normal(d)).astype(np.float32)
        pos = rng.integers(0, 3000, (7, 1)).astype(np.int32)
        got = oracle.norm_rope(x, w, rot, theta, 1e-6, np.broadcast_to(pos, (7, 3)))
        want = numpy_norm_rope(x, w, rot, theta, 1e-6, np.broadcast_to(pos, (7, 3)))
        # f32 angles: pos * ulp(1) = 3000 * 6e-8 = 2e-4 rad at the fastest pair
        assert np.abs(got - want).max() < 1e-3 * np.abs(want).max()
