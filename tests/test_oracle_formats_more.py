"""Pins the oracle's other block formats (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K) without restating its code:
the exact rational value of every element, written here from the format descriptions
(tensor/internal/cpu/kernels/quantized.go:13-82 and the dequantize kernels of
tensor/internal/cuda/kernels/quantized.cu), against the oracle's f32 result (one rounding of it, or none),
and the oracle's vec-dots against the exact sum of products.
"""
from fractions import Fraction

import numpy as np
import pytest

from candy_amd import synth
from oracle import oracle as o

Q8_0 = synth.Q8_0
Q4_1, Q4_1_GGML, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K = (synth.Q4_1, synth.Q4_1_GGML, synth.Q5_0, synth.Q5_1, synth.Q2_K,
                                                      synth.Q3_K, synth.Q5_K, synth.Q8_K)
NEW = [Q4_1, Q4_1_GGML, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K]
SPECIAL = [0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF, 0x3C00, 0x2000, 0x251F]


def half_fraction(bits: int) -> Fraction:
    return Fraction(float(np.array([bits], np.uint16).view(np.float16)[0]))


def frac_to_f32(fr: Fraction) -> np.float32:
    """Round an exact rational to binary32, nearest-even, without going through a double."""
    if fr == 0:
        return np.float32(0.0)
    sign = -1 if fr < 0 else 1
    a = abs(fr)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    e = max(e, -126)
    scaled = a / (Fraction(2) ** (e - 23))
    q, r = divmod(scaled.numerator, scaled.denominator)
    if 2 * r > scaled.denominator or (2 * r == scaled.denominator and (q & 1)):
        q += 1
    return np.float32(sign * float(Fraction(q) * Fraction(2) ** (e - 23)))


def k4(scales12) -> tuple[list[int], list[int]]:
    """6-bit (scale, min) of the eight sub-blocks from the 12 packed bytes (layout of quantized.cu:993-1005)."""
    s = [int(v) for v in scales12]
    sc = [s[j] & 63 for j in range(4)] + [(s[j + 4] & 0xF) | ((s[j - 4] >> 6) << 4) for j in range(4, 8)]
    mn = [s[j + 4] & 63 for j in range(4)] + [(s[j + 4] >> 4) | ((s[j] >> 6) << 4) for j in range(4, 8)]
    return sc, mn


def exact_block(fmt: int, blk) -> list[Fraction]:
    """Exact value of every element of one block, in element order."""
    if fmt in (Q4_1, Q4_1_GGML):
        d, m = half_fraction(int(blk["d"])), half_fraction(int(blk["m"]))
        out = [Fraction(0)] * 32
        for j in range(16):
            lo, hi = int(blk["qs"][j]) & 15, int(blk["qs"][j]) >> 4
            i_lo, i_hi = (2 * j, 2 * j + 1) if fmt == Q4_1 else (j, j + 16)
            out[i_lo], out[i_hi] = d * lo + m, d * hi + m
        return out
    if fmt in (Q5_0, Q5_1):
        qh = int.from_bytes(bytes(blk["qh"]), "little")
        lev = [((int(blk["qs"][e % 16]) >> (4 if e >= 16 else 0)) & 15) | (((qh >> e) & 1) << 4) for e in range(32)]
        d = half_fraction(int(blk["d"]))
        if fmt == Q5_0:
            return [d * (v - 16) for v in lev]
        m = half_fraction(int(blk["m"]))
        return [d * v + m for v in lev]
    if fmt == Q2_K:
        d, dmin = half_fraction(int(blk["d"])), half_fraction(int(blk["dmin"]))
        out = []
        for e in range(256):
            n, k, l = e // 128, (e % 128) // 32, e % 32
            sc = int(blk["scales"][e // 16])
            out.append(d * (sc & 15) * ((int(blk["qs"][32 * n + l]) >> (2 * k)) & 3) - dmin * (sc >> 4))
        return out
    if fmt == Q3_K:
        d = half_fraction(int(blk["d"]))
        s = [int(v) for v in blk["scales"]]
        # 16 six-bit scales: low 4 bits in the nibbles of bytes 0..7, high 2 bits in the bit pairs of bytes 8..11
        sc = [((s[i % 8] >> (4 * (i // 8))) & 15) | (((s[8 + i % 4] >> (2 * (i // 4))) & 3) << 4) for i in range(16)]
        out = []
        for e in range(256):
            n, j, l = e // 128, (e % 128) // 32, e % 32
            lev = ((int(blk["qs"][32 * n + l]) >> (2 * j)) & 3) - (0 if (int(blk["hmask"][l]) >> (4 * n + j)) & 1 else 4)
            out.append(d * (sc[e // 16] - 32) * lev)
        return out
    if fmt == Q5_K:
        d, dmin = half_fraction(int(blk["d"])), half_fraction(int(blk["dmin"]))
        sc, mn = k4(blk["scales"])
        out = []
        for e in range(256):
            t, l = e // 32, e % 32
            q = int(blk["qs"][32 * (t // 2) + l])
            lev = ((q >> 4) if t & 1 else (q & 15)) + (16 if (int(blk["qh"][l]) >> t) & 1 else 0)
            out.append(d * sc[t] * lev - dmin * mn[t])
        return out
    if fmt == Q8_K:
        d = Fraction(float(blk["d"]))
        return [d * int(q) for q in blk["qs"]]
    raise AssertionError(fmt)


def test_block_sizes():
    # quantized.cu static_asserts: 20 / 22 / 24 bytes, q2_K 84, q3_K 110, q5_K 176, q8_K 292
    assert [o.block_bytes(f) for f in NEW] == [20, 20, 22, 24, 84, 110, 176, 292]
    assert [o.block_elems(f) for f in NEW] == [32, 32, 32, 32, 256, 256, 256, 256]


@pytest.mark.parametrize("fmt", NEW, ids=lambda f: synth.FORMAT_NAMES[f])
def test_dequantize_is_the_exact_value_rounded_once(fmt):
    n = 14
    dt = synth.BLOCK_DTYPES[fmt]
    blocks = synth.random_blocks(fmt, n, seed=30 + fmt).view(dt).copy()
    if fmt != Q8_K:
        for i, s in enumerate(SPECIAL):
            blocks["d"][i] = s
            for other in ("m", "dmin"):
                if other in dt.names:
                    blocks[other][i] = SPECIAL[(3 * i + 1) % len(SPECIAL)]
    y = o.dequantize(fmt, blocks).reshape(n, -1)
    for b in range(n):
        want = exact_block(fmt, blocks[b])
        for e, fr in enumerate(want):
            assert y[b, e] == frac_to_f32(fr), (synth.FORMAT_NAMES[fmt], b, e)


def test_q4_1_orders_are_a_permutation_of_each_other():
    blocks = synth.random_blocks(Q4_1, 9, seed=2)
    a = o.dequantize(Q4_1, blocks).reshape(-1, 32)
    g = o.dequantize(Q4_1_GGML, blocks).reshape(-1, 32)
    assert np.array_equal(a[:, 0::2], g[:, :16]) and np.array_equal(a[:, 1::2], g[:, 16:])


def test_q3_k_values_need_no_rounding():
    blocks = synth.random_blocks(Q3_K, 6, seed=3).view(synth.BLOCK_DTYPES[Q3_K])
    y = o.dequantize(Q3_K, blocks).reshape(6, 256)
    for b in range(6):
        assert [Fraction(float(v)) for v in y[b]] == exact_block(Q3_K, blocks[b])


@pytest.mark.parametrize("fmt", [f for f in NEW if f != Q8_K], ids=lambda f: synth.FORMAT_NAMES[f])
def test_vec_dot_equals_exact_sum_of_products(fmt):
    k, rows = 512, 5
    w = synth.random_weight(fmt, rows, k, seed=100 + fmt, scale=synth.unit_scale(fmt))
    x = synth.random_activations(1, k, seed=200 + fmt)
    xq = o.quantize_q8_0(x)
    xb = xq.view(synth.BLOCK_DTYPES[Q8_0])
    xv = [half_fraction(int(b["d"])) * int(q) for b in xb for q in b["qs"]]
    rb = synth.weight_nbytes(fmt, 1, k)
    for r in range(rows):
        wrow = w[r * rb:(r + 1) * rb]
        wv = [v for blk in wrow.view(synth.BLOCK_DTYPES[fmt]) for v in exact_block(fmt, blk)]
        exact = sum((a * b for a, b in zip(wv, xv)), Fraction(0))
        mass = float(sum(abs(a * b) for a, b in zip(wv, xv)))
        got = o.vec_dot_q8_0(fmt, wrow, xq, k)
        assert abs(Fraction(got) - exact) <= Fraction(2e-6) * Fraction(mass) + Fraction(1e-30), (fmt, r)


def test_q8_k_has_no_weight_vec_dot():
    w = synth.random_weight(Q8_K, 1, 256, seed=1)
    xq = o.quantize_q8_0(synth.random_activations(1, 256, seed=2))
    assert np.isnan(o.vec_dot_q8_0(Q8_K, w, xq, 256))


# ---------------------------------------------------------------------- the other dequantize outputs
def test_f64_twins_are_the_exact_values_rounded_once():
    # quantized.go:96-104, 119-128, 139-144.  Exact rational value of each element -> nearest double must be what the
    # oracle returns; a dropped "- 8", a swapped nibble or the min taken from the wrong half fails.  For Q4_0 and Q8_0
    # the product fits 24 bits, so the float64 twin is also the f32 output widened.
    rng = np.random.default_rng(5)
    for fmt, width in ((synth.Q4_0, 18), (Q4_1, 20), (Q8_0, 34)):
        blocks = rng.integers(0, 256, (40, width), dtype=np.uint8)
        for i, h in enumerate(SPECIAL):           # special scale values, and a finite min for Q4_1
            blocks[i, 0], blocks[i, 1] = h & 0xFF, h >> 8
        blocks[:, 1] &= 0x7B                       # keep d finite
        if fmt == Q4_1:
            blocks[:, 3] &= 0x7B
        got = o.dequantize_f64(fmt, blocks)
        for b in range(blocks.shape[0]):
            d = half_fraction(int(blocks[b, 0]) | int(blocks[b, 1]) << 8)
            for e in range(32):
                if fmt == synth.Q4_0:
                    q = (int(blocks[b, 2 + e // 2]) >> (4 * (e & 1))) & 15
                    exact = d * (q - 8)
                elif fmt == Q4_1:
                    q = (int(blocks[b, 4 + e // 2]) >> (4 * (e & 1))) & 15
                    exact = d * q + half_fraction(int(blocks[b, 2]) | int(blocks[b, 3]) << 8)
                else:
                    exact = d * int(np.int8(blocks[b, 2 + e]))
                assert got[b * 32 + e] == float(exact), (fmt, b, e)   # float(Fraction) rounds to nearest even
        if fmt != Q4_1:
            assert np.array_equal(got, o.dequantize(fmt, blocks).astype(np.float64))


def test_f16_output_is_the_f32_output_rounded_to_nearest_even():
    # kernels.go:486-505: same kernels with dst_t = half.  Checked against the exact value rounded by hand for the
    # 32-value formats (one rounding when the f32 value is exact, which it is for Q4_0 / Q8_0: at most 19 bits)
    rng = np.random.default_rng(6)
    for fmt, width in ((synth.Q4_0, 18), (Q8_0, 34)):
        blocks = rng.integers(0, 256, (64, width), dtype=np.uint8)
        blocks[:, 1] &= 0x3F                       # |d| < 2: products stay inside fp16's range
        got = o.dequantize_f16(fmt, blocks)
        assert got.dtype == np.float16
        for b in range(0, 64, 7):
            d = half_fraction(int(blocks[b, 0]) | int(blocks[b, 1]) << 8)
            for e in range(32):
                q = ((int(blocks[b, 2 + e // 2]) >> (4 * (e & 1))) & 15) - 8 if fmt == synth.Q4_0 else int(np.int8(blocks[b, 2 + e]))
                exact = d * q
                lo, hi = np.float16(float(exact)), got[b * 32 + e]
                # float(exact) is exact here (19 bits), and numpy's float64 -> float16 is round to nearest even
                assert lo == hi or (np.isnan(lo) and np.isnan(hi)), (fmt, b, e)
