"""Hand-computed q4_0 blocks: inputs and the bytes ggml's published rule gives for them.

The rule (llama.cpp ggml-quants.c, quantize_row_q4_0_ref, which engine/core/gguf_quant.cpp:1 cites for its block
formats): `max` is the FIRST element of largest magnitude, sign kept; d = max / -8; id = 1 / d (0 if d == 0);
code = min(15, trunc(x * id + 8.5)); byte j = code[j] | code[j + 16] << 4; the scale is stored as f16(d).
Every expected byte below was worked out on paper from that text, not by running any implementation:
  * with max = -8 the scale is +1 and x * id = x, so code = trunc(x + 8.5): halves go UP (-0.5 -> 8, 0.5 -> 9,
    -1.5 -> 7, 1.5 -> 10), 7.5 and 8 clip at 15, zero is code 8;
  * with max = +8 the scale is -1 and x * id = -x;
  * of +8 and -8 in one block the earlier one decides the sign of the scale.
An implementation that rounds halves away from zero, takes the last of two equal magnitudes, or forgets the clip
fails at least one block.
"""
import numpy as np

F16_ONE, F16_MINUS_ONE = 0x3C00, 0xBC00


def _pack(codes):
    codes = np.asarray(codes, np.uint8)
    return (codes[:16] | (codes[16:] << 4)).astype(np.uint8)


def _block(scale_bits, codes):
    return np.concatenate([np.array([scale_bits & 0xFF, scale_bits >> 8], np.uint8), _pack(codes)])


def known_answers():
    """(x f32 [n][32], expected blocks u8 [n][18], names)."""
    xs, want, names = [], [], []

    def add(name, x, scale_bits, codes):
        assert len(x) == 32 and len(codes) == 32
        xs.append(np.asarray(x, np.float32)), want.append(_block(scale_bits, codes)), names.append(name)

    # 1. ties and the clip, scale +1 (the -8 comes first, so the later +8 does not take over)
    x = [0.0] * 32
    c = [8] * 32
    x[:8] = [-8, .5, -.5, 1.5, -1.5, 7, 7.5, 8]
    c[:8] = [0, 9, 8, 10, 7, 15, 15, 15]
    add("ties d=+1", x, F16_ONE, c)
    # 2. every half k + 0.5, k = -8 .. 7, in the high-nibble half of the block; scale +1
    x = [0.0] * 32
    c = [8] * 32
    x[0], c[0] = -8, 0
    for i, k in enumerate(range(-8, 8)):
        x[16 + i] = k + 0.5
        c[16 + i] = min(15, k + 9)           # trunc(k + 0.5 + 8.5) = k + 9
    add("all halves d=+1", x, F16_ONE, c)
    # 3. scale -1 (+8 first): x * id = -x
    x = [0.0] * 32
    c = [8] * 32
    x[:8] = [8, -8, .5, -.5, 1.5, -1.5, -7, -7.5]
    c[:8] = [0, 15, 8, 9, 7, 10, 15, 15]     # -8 -> 8 + 8.5 = 16.5 -> clip 15; .5 -> 8.0; -.5 -> 9.0; -7 -> 15.5; -7.5 -> 16 -> 15
    add("ties d=-1", x, F16_MINUS_ONE, c)
    # 4. the first of two equal magnitudes decides, wherever the two sit: +8 at p, -8 at p2 > p, and the mirror image.
    # (In the GPU append a block lies across 8 lanes, 4 dims each: p and p2 run over all lanes and slots.)
    for p in range(32):
        for p2 in range(p + 1, 32):
            x = [0.0] * 32
            c = [8] * 32
            x[p], x[p2] = 8, -8
            c[p], c[p2] = 0, 15
            add(f"+8@{p} -8@{p2}", x, F16_MINUS_ONE, c)
            x = [0.0] * 32
            c = [8] * 32
            x[p], x[p2] = -8, 8
            c[p], c[p2] = 0, 15
            add(f"-8@{p} +8@{p2}", x, F16_ONE, c)
    # 5. a smaller magnitude never wins, before or after: -4 .. 8 .. -7.99 -> scale -1, codes from -x
    for p in range(32):
        x = [0.0] * 32
        c = [8] * 32
        x[p], c[p] = 8, 0
        x[(p + 1) % 32], c[(p + 1) % 32] = -4, 12       # 4 + 8.5 -> 12
        x[(p + 31) % 32], c[(p + 31) % 32] = -7.75, 15  # 7.75 + 8.5 = 16.25 -> 16 -> clip 15
        add(f"max@{p} with smaller neighbours", x, F16_MINUS_ONE, c)
    # 6. a scale that is not a power of two: max = -6 -> d = 0.75 (f16 0x3A00), id = 4/3 rounded to f32;
    # x = 0.75 k are exact multiples: 0.75 k * f32(4/3) lies within 1e-7 of k, so trunc(. + 8.5) = k + 8
    x = [0.0] * 32
    c = [8] * 32
    for i, k in enumerate(range(-8, 8)):
        x[i] = 0.75 * k
        c[i] = k + 8
    add("d=0.75", x, 0x3A00, c)
    # 7. the all-zero block: d = 0 / -8 = -0.0 (f16 0x8000), id = 0, every code 8
    add("zeros", [0.0] * 32, 0x8000, [8] * 32)
    return np.stack(xs), np.stack(want), names
