"""The CPU oracle's block arithmetic against the reference's own compiled code (golden vectors made with
engine/core/gguf_quant.cpp, and oracle/_ref directly where it is built) and against what the mathematics fixes."""
import numpy as np
import pytest

import oracle


def f16_of(bits):
    return np.asarray(bits, np.uint16).view(np.float16)


def test_q8_0_quantize_matches_reference_golden(golden):
    got = oracle.quantize_q8_0(golden["q8_in"])
    assert np.array_equal(got, golden["q8_out"])


def test_dequantize_matches_reference_golden(golden):
    assert np.array_equal(oracle.dequantize_q8_0(golden["d8_in"]).view(np.uint32),
                          golden["d8_out"].reshape(-1).view(np.uint32))
    assert np.array_equal(oracle.dequantize_q4_0(golden["d4_in"]).view(np.uint32),
                          golden["d4_out"].reshape(-1).view(np.uint32))


@pytest.mark.skipif(oracle.ref() is None, reason="oracle/_ref not built (no reference tree here)")
def test_q8_0_quantize_matches_reference_live():
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((4096, 32)) * 10.0 ** rng.uniform(-3, 3, (4096, 1))).astype(np.float32)
    assert np.array_equal(oracle.quantize_q8_0(x), oracle.ref_quantize_q8_0(x))
    b = oracle.quantize_q8_0(x)
    assert np.array_equal(oracle.dequantize_q8_0(b), oracle.ref_dequantize_q8_0(b))


@pytest.mark.skipif(oracle.ref() is None, reason="oracle/_ref not built (no reference tree here)")
def test_half_conversions_match_reference_live():
    bits = np.arange(65536, dtype=np.uint16)
    a, b = oracle.f16_bits_to_f32(bits), oracle.ref_f16_bits_to_f32(bits)
    nan = np.isnan(b)
    assert np.array_equal(np.isnan(a), nan) and np.array_equal(a[~nan].view(np.uint32), b[~nan].view(np.uint32))
    a, b = oracle.bf16_bits_to_f32(bits), oracle.ref_bf16_bits_to_f32(bits)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


def test_f16_to_f32_all_patterns_against_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    want = f16_of(bits).astype(np.float32)
    got = oracle.f16_bits_to_f32(bits)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_bf16_to_f32_all_patterns():
    bits = np.arange(65536, dtype=np.uint16)
    want = (bits.astype(np.uint32) << 16).view(np.float32)
    assert np.array_equal(oracle.bf16_bits_to_f32(bits).view(np.uint32), want.view(np.uint32))


def test_f32_to_f16_against_numpy():
    rng = np.random.default_rng(3)
    # every f16 value, the midpoints between neighbours (ties), one ulp either side of them, and random f32 bits
    h = np.arange(0x7C00, dtype=np.uint16)
    v = f16_of(h).astype(np.float64)
    mid = ((v[:-1] + v[1:]) / 2).astype(np.float32)
    xs = [f16_of(h).astype(np.float32), mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
          np.array([65504, 65519.99, 65520, 65536, 1e9, np.inf, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0000001, 2.0 ** -26,
                    0.0, 1e-45], np.float32),
          rng.integers(0, 2 ** 32, 400000, dtype=np.uint64).astype(np.uint32).view(np.float32)]
    x = np.concatenate(xs)
    x = np.concatenate([x, -x])
    x = x[~np.isnan(x)]
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(x), want)


def test_f32_to_bf16_round_to_nearest_even():
    rng = np.random.default_rng(4)
    x = rng.integers(0, 2 ** 32, 300000, dtype=np.uint64).astype(np.uint32).view(np.float32)
    x = x[np.isfinite(x)]
    got = oracle.bf16_bits_to_f32(oracle.f32_to_bf16_bits(x)).astype(np.float64)
    lo = (x.view(np.uint32) & 0xFFFF0000).view(np.float32).astype(np.float64)           # truncation toward zero
    hi = ((x.view(np.uint32) & 0xFFFF0000) + 0x10000).view(np.float32).astype(np.float64)  # next bf16 away from zero
    xd = x.astype(np.float64)
    with np.errstate(invalid="ignore", over="ignore"):
        nearest = np.where(np.abs(xd - lo) < np.abs(hi - xd), lo, hi)
        tie = np.abs(xd - lo) == np.abs(hi - xd)
        even = np.where((x.view(np.uint32) >> 16) & 1, hi, lo)
        want = np.where(tie, even, nearest)
    ok = np.isfinite(hi)
    assert np.array_equal(got[ok], want[ok])


def test_q8_0_invariants():
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((2048, 32)) * 10.0 ** rng.uniform(-2, 2, (2048, 1))).astype(np.float32)
    b = oracle.quantize_q8_0(x)
    codes = b[:, 2:].view(np.int8).astype(np.int32)
    amax_idx = np.abs(x).argmax(1)
    assert np.all(np.abs(codes[np.arange(len(x)), amax_idx]) == 127)       # the amax element hits +-127
    assert codes.min() >= -127 and codes.max() <= 127
    d32 = (np.abs(x).max(1) / np.float32(127)).astype(np.float32)
    assert np.array_equal(b[:, :2].copy().view(np.uint16).reshape(-1), d32.astype(np.float16).view(np.uint16))
    # |x - d32 * code| <= d32 / 2 (+ rounding of x * inv), and with the stored f16 scale + |x| 2^-11
    err = np.abs(x - d32[:, None] * codes)
    assert np.all(err <= d32[:, None] * 0.5000005)
    d16 = b[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    y = oracle.dequantize_q8_0(b).reshape(-1, 32)
    assert np.array_equal(y, d16[:, None] * codes.astype(np.float32))
    assert np.all(np.abs(y - x) <= d32[:, None] * 0.5000005 + np.abs(x) * 2.0 ** -11 + 1e-30)


def test_q8_0_idempotent_when_scale_is_f16_exact():
    rng = np.random.default_rng(6)
    codes = rng.integers(-127, 128, (512, 32)).astype(np.float32)
    codes[:, 0] = 127
    d = (2.0 ** rng.integers(-10, 6, (512, 1))).astype(np.float32)         # f16-exact scales
    b = oracle.quantize_q8_0(codes * d)
    assert np.array_equal(oracle.quantize_q8_0(oracle.dequantize_q8_0(b)), b)
    assert np.array_equal(b[:, 2:].view(np.int8), codes.astype(np.int8))


def test_q8_0_halves_round_away_from_zero():
    x = np.zeros(32, np.float32)
    x[:7] = [127, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5]
    c = oracle.quantize_q8_0(x)[0, 2:].view(np.int8)
    assert list(c[:7]) == [127, 1, 2, 3, -1, -2, -3]


def test_q4_0_invariants():
    """q4_0 quantize is not pinned by the reference (it has none): ggml's rule, checked by what it guarantees."""
    rng = np.random.default_rng(8)
    x = (rng.standard_normal((2048, 32)) * 10.0 ** rng.uniform(-2, 2, (2048, 1))).astype(np.float32)
    x[:256, 5] *= 20                                                         # outlier channel, as config 5 has
    b = oracle.quantize_q4_0(x)
    lo, hi = (b[:, 2:] & 0xF).astype(np.int32), (b[:, 2:] >> 4).astype(np.int32)
    codes = np.concatenate([lo, hi], 1)                                       # element j low nibble, j + 16 high
    assert codes.min() >= 0 and codes.max() <= 15
    idx = np.abs(x).argmax(1)
    assert np.all(codes[np.arange(len(x)), idx] == 0)                         # largest magnitude -> code 0 = -8 d
    d32 = (x[np.arange(len(x)), idx] / np.float32(-8)).astype(np.float32)
    assert np.array_equal(b[:, :2].copy().view(np.uint16).reshape(-1), d32.astype(np.float16).view(np.uint16))
    y32 = d32[:, None] * (codes - 8)
    clip = codes == 15                                                        # +8 d is not representable: clipped at +7 d
    err = np.abs(x - y32)
    assert np.all(err[~clip] <= np.abs(d32)[:, None].repeat(32, 1)[~clip] * 0.5000005)
    assert np.all(err[clip] <= np.abs(d32)[:, None].repeat(32, 1)[clip] * 1.0000005)
    d16 = b[:, :2].copy().view(np.float16).astype(np.float32).reshape(-1)
    assert np.array_equal(oracle.dequantize_q4_0(b).reshape(-1, 32), d16[:, None] * (codes - 8).astype(np.float32))
    z = oracle.quantize_q4_0(np.zeros(32, np.float32))
    assert np.array_equal(z[0], np.array([0, 0x80] + [0x88] * 16, np.uint8))  # all-zero block: d = 0 / -8 = -0.0, codes 8


def test_q4_0_known_answers():
    """ggml's quantize_row_q4_0_ref on hand-computed blocks (tests/q4_known_answers.py): halves round up, the clip at
    code 15, the first of two equal magnitudes decides the scale's sign, for every pair of positions in a block."""
    from q4_known_answers import known_answers
    x, want, names = known_answers()
    got = oracle.quantize_q4_0(x)
    for i in np.flatnonzero((got != want).any(1)):
        raise AssertionError(f"block '{names[i]}': got {got[i].tolist()}, want {want[i].tolist()}")
    # and what those blocks decode to, worked out the same way: (code - 8) * d
    y = oracle.dequantize_q4_0(want[:1]).reshape(32)
    assert list(y[:8]) == [-8, 1, 0, 2, -1, 7, 7, 7] and not y[8:].any()
    y = oracle.dequantize_q4_0(want[2:3]).reshape(32)
    assert list(y[:8]) == [8, -7, 0, -1, 1, -2, -7, -7]


def test_the_kernels_rounding_is_lround_for_every_float_a_code_can_come_from():
    """The append kernels round x * inv as trunc(r + copysign(0.5 - 2^-25, r)) where the reference calls lround
    (gguf_quant.cpp:316); codes come from |r| <= 128 (anything larger becomes 0 on both sides). Every float up to
    129, both signs, 2.2e9 values."""
    last = int(np.array([129.0], np.float32).view(np.uint32)[0])
    assert oracle.lround_identity_mismatches(0, last) == 0
    # the identity is not a tautology: with 0.5 itself the float below one half goes wrong
    below_half = np.array([0.5], np.float32).view(np.uint32)[0] - 1
    r = np.array([below_half], np.uint32).view(np.float32)[0]
    assert int(np.float32(r) + np.float32(0.5)) == 1 and round(float(r)) == 0
