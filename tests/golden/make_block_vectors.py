#!/usr/bin/env python3
"""Writes tests/golden/block_vectors.npz: inputs and the outputs of the REFERENCE's own compiled block code
(oracle/_ref/libref.so = engine/core/gguf_quant.cpp built from /root/reference by oracle/Makefile).

Run in the authoring container, where the reference tree exists:  python tests/golden/make_block_vectors.py
The .npz holds data only (plain arrays, loaded with allow_pickle=False):
  q8_in  f32 [n][32]   q8_out u8 [n][34]   yah::core::QuantizeQ8_0 (gguf_quant.cpp:310-320)
  d8_in  u8 [n][34]    d8_out f32 [n][32]  Dequantize(kQ8_0)        (gguf_quant.cpp:72-75)
  d4_in  u8 [n][18]    d4_out f32 [n][32]  Dequantize(kQ4_0)        (gguf_quant.cpp:48-51)
"""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", ".."))
import oracle  # noqa: E402


def q8_inputs():
    rng = np.random.default_rng(20240601)
    rows = [rng.standard_normal((256, 32)).astype(np.float32)]                  # the configs' N(0,1) sources
    rows.append((rng.standard_normal((64, 32)) * 10.0 ** rng.uniform(-6, 4, (64, 1))).astype(np.float32))
    rows.append(np.zeros((1, 32), np.float32))                                   # d = 0, inv = 0, codes 0
    one = np.zeros((1, 32), np.float32)
    one[0, 7] = -3.25                                                            # single outlier
    rows.append(one)
    # amax = 127 -> d = 1, inv = 1: halves sit exactly on a code boundary; lround goes away from zero, rne would not
    h = np.zeros((1, 32), np.float32)
    h[0, 0] = 127.0
    h[0, 1:21] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 63.5, -63.5, 126.5, -126.5, 0.49999997, -0.49999997,
                  1.4999999, 2.5000002, 125.5, -125.5, 100.5, -100.5, 0.0, -0.0]
    rows.append(h)
    rows.append(-h)
    # amax that f16 holds exactly (d = 2^-3) and one it does not
    e = np.zeros((2, 32), np.float32)
    e[0, :4] = [127 * 0.125, 0.125 * 3.5, -0.125 * 4.5, 0.0625]
    e[1, :4] = [0.1, 0.05, -0.033, 0.0999]
    rows.append(e)
    # tiny scales: d below the f16 subnormal range (stored scale 0, codes still non-zero), f32-subnormal d,
    # and d so small that 1/d overflows (the codes of such a block are whatever lround(inf / nan) gives: 0 on x86-64)
    t = np.zeros((4, 32), np.float32)
    t[0, :3] = [1e-9, -5e-10, 2.5e-10]
    t[1, :3] = [1e-36, -5e-37, 1e-38]
    t[2, :3] = [1e-38, -5e-39, 1e-39]
    t[3, :3] = [1e-40, -5e-41, 0]
    rows.append(t)
    big = np.zeros((2, 32), np.float32)
    big[0, :3] = [65504.0 * 127, 1e6, -3e6]      # d = 65504, the largest finite f16
    big[1, :3] = [1e7, -1e7, 5e6]                # d rounds to f16 inf
    rows.append(big)
    # bf16- and f16-representable sources (what the append reads), widened exactly
    b = rng.standard_normal((64, 32)).astype(np.float32)
    rows.append((b.view(np.uint32) & 0xFFFF0000).view(np.float32))
    rows.append(rng.standard_normal((64, 32)).astype(np.float16).astype(np.float32))
    return np.concatenate(rows, 0)


def main():
    if oracle.ref() is None:
        oracle.build()
    if oracle.ref() is None:
        raise SystemExit("oracle/_ref/libref.so is not built (needs /root/reference and amdclang++)")
    rng = np.random.default_rng(7)
    q8_in = q8_inputs()
    q8_out = oracle.ref_quantize_q8_0(q8_in)
    # dequantizers: random code bytes, scales drawn from finite f16 bit patterns (incl. subnormals, +-0)
    def blocks(bb, n):
        b = rng.integers(0, 256, (n, bb), dtype=np.uint8)
        s = rng.integers(0, 0x7C00, n).astype(np.uint16) | (rng.integers(0, 2, n).astype(np.uint16) << 15)
        s[:4] = [0, 0x8000, 1, 0x03FF]
        b[:, :2] = s.view(np.uint8).reshape(n, 2)
        return b
    d8_in, d4_in = blocks(34, 192), blocks(18, 192)
    d8_out = oracle.ref_dequantize_q8_0(d8_in).reshape(-1, 32)
    d4_out = oracle.ref_dequantize_q4_0(d4_in).reshape(-1, 32)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "block_vectors.npz")
    np.savez_compressed(out, q8_in=q8_in, q8_out=q8_out, d8_in=d8_in, d8_out=d8_out, d4_in=d4_in, d4_out=d4_out)
    print(out, os.path.getsize(out), "bytes;", len(q8_in), "q8 blocks")


if __name__ == "__main__":
    main()
