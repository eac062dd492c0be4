"""Pins the CPU oracle's block-format functions with checks that do not restate its code:
IEEE conversions against numpy, dequantized values against exact rational arithmetic,
the 6-bit scale unpack against the reference's other (16-bit masked) encoding of the same
bits, the quantizer against a float64 evaluation, and the vec-dots against exact sums.
"""
from fractions import Fraction

import numpy as np
import pytest

from candy_amd import synth
from oracle import oracle as o

Q4_0, Q8_0, Q4_K, Q6_K, Q4_0_GGML = synth.Q4_0, synth.Q8_0, synth.Q4_K, synth.Q6_K, synth.Q4_0_GGML


# ---------------------------------------------------------------- helpers (independent of the oracle)

def half_fraction(bits: int) -> Fraction:
    """Exact value of a finite fp16 bit pattern (numpy decodes it)."""
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
    scaled = a / (Fraction(2) ** (e - 23))  # significand as a rational in [2^23, 2^24) (or less, subnormal)
    q, r = divmod(scaled.numerator, scaled.denominator)
    twice = 2 * r
    if twice > scaled.denominator or (twice == scaled.denominator and (q & 1)):
        q += 1
    return np.float32(sign * float(Fraction(q) * Fraction(2) ** (e - 23)))


def k4_from_masked_u16(scales12: np.ndarray):
    """Scale/min unpack as the vec-dot does it on 16-bit words
    (tensor/internal/cuda/kernels/quantized.cu:2600-2612)."""
    s16 = scales12.view("<u2")
    sc, mn = [0] * 8, [0] * 8
    for j in range(4):  # j = pair of sub-blocks (2j, 2j+1)
        if j < 2:
            a0 = int(s16[j]) & 0x3F3F
            a1 = int(s16[j + 2]) & 0x3F3F
        else:
            a0 = (int(s16[j + 2]) & 0x0F0F) | ((int(s16[j - 2]) & 0xC0C0) >> 2)
            a1 = ((int(s16[j + 2]) >> 4) & 0x0F0F) | ((int(s16[j]) & 0xC0C0) >> 2)
        sc[2 * j], sc[2 * j + 1] = a0 & 0xFF, a0 >> 8
        mn[2 * j], mn[2 * j + 1] = a1 & 0xFF, a1 >> 8
    return sc, mn


def q6_quant(blk, e: int) -> int:
    """6-bit quant of element e of a Q6_K super-block, minus 32 (written from the format
    description: 4 low bits in ql, 2 high bits in qh, 128-element halves, 32-element quarters)."""
    half, rem = divmod(e, 128)
    quarter, il = divmod(rem, 32)
    byte = int(blk["ql"][64 * half + 32 * (quarter & 1) + il])
    lo4 = (byte >> 4) if quarter >= 2 else (byte & 15)
    hi2 = (int(blk["qh"][32 * half + il]) >> (2 * quarter)) & 3
    return (lo4 | (hi2 << 4)) - 32


def q4k_quant(blk, e: int) -> int:
    t, l = divmod(e, 32)
    byte = int(blk["qs"][32 * (t // 2) + l])
    return (byte >> 4) if (t & 1) else (byte & 15)


# ---------------------------------------------------------------- struct sizes

def test_block_sizes_match_reference_asserts():
    # quantized.cu:305,347,410,444 assert 18 / 34 / 144 / 210 bytes
    assert [o.block_bytes(f) for f in (Q4_0, Q8_0, Q4_K, Q6_K)] == [18, 34, 144, 210]
    assert [o.block_elems(f) for f in (Q4_0, Q8_0, Q4_K, Q6_K)] == [32, 32, 256, 256]
    assert o.block_bytes(9999) == 0 and o.block_elems(9999) == 0
    for f in (Q4_0, Q8_0, Q4_K, Q6_K):
        assert synth.BLOCK_BYTES[f] == o.block_bytes(f)


# ---------------------------------------------------------------- fp16 <-> f32

def test_fp16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32).view(np.uint32)
    got = np.array([np.float32(o.fp16_to_f32(int(b))).view(np.uint32) for b in bits], np.uint32)
    nan = np.isnan(bits.view(np.float16))
    assert np.array_equal(got[~nan], want[~nan])
    # NaN: payload shifted up by 13, sign kept (quantized.go:156). The quiet bit is left out of the
    # comparison: returning a float through the C ABI may quieten a signalling NaN.
    assert np.all(np.isnan(got[nan].view(np.float32)))
    b32 = bits[nan].astype(np.uint32)
    assert np.array_equal(got[nan] & 0x803FE000, ((b32 & 0x8000) << 16 | (b32 & 0x3FF) << 13) & 0x803FE000)


def _check_f32_to_fp16(vals: np.ndarray):
    vals = vals.astype(np.float32)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([o.f32_to_fp16(float(v)) for v in vals], np.uint16)
    nan = np.isnan(vals)
    assert np.array_equal(got[~nan], want[~nan])
    assert np.all(np.isnan(got[nan].view(np.float16)))


def test_f32_to_fp16_roundtrip_all_halves():
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    _check_f32_to_fp16(bits.view(np.float16).astype(np.float32))


def test_f32_to_fp16_midpoints_and_neighbours():
    # all finite non-negative halves, midpoints between neighbours, and one f32 ulp either side
    h = np.arange(0, 0x7C00, dtype=np.uint16).view(np.float16).astype(np.float32)
    mid = (h[:-1].astype(np.float64) + h[1:].astype(np.float64)) / 2  # exact in f32
    mid = mid.astype(np.float32)
    cand = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)), np.nextafter(mid, np.float32(-np.inf)),
                           np.array([65504, 65519.996, 65520, 65536, 1e9, 2.0 ** -25, 2.0 ** -24, 5.9e-8, 3e-8, 2.98e-8], np.float32)])
    _check_f32_to_fp16(np.concatenate([cand, -cand]))


def test_f32_to_fp16_random_bit_patterns():
    rng = np.random.default_rng(7)
    _check_f32_to_fp16(rng.integers(0, 2 ** 32, 200_000, dtype=np.uint64).astype(np.uint32).view(np.float32))


# ---------------------------------------------------------------- dequantize

def _special_scales():
    # zero, subnormals, smallest/largest normals, both signs
    return [0x0000, 0x8000, 0x0001, 0x03FF, 0x0400, 0x7BFF, 0xFBFF, 0x3C00, 0x2000, 0x251F]


def test_dequant_q4_0_exact_and_interleaved():
    blocks = synth.random_blocks(Q4_0, 64, seed=1).view(synth.BLOCK_DTYPES[Q4_0]).copy()
    for i, s in enumerate(_special_scales()):
        blocks["d"][i] = s
    y = o.dequantize(Q4_0, blocks).reshape(-1, 32)
    for b in range(len(blocks)):
        d = half_fraction(int(blocks["d"][b]))
        for j in range(16):
            lo, hi = int(blocks["qs"][b][j]) & 15, int(blocks["qs"][b][j]) >> 4
            # candy CPU order (quantized.go:87-92): 2j <- low nibble, 2j+1 <- high nibble; value exact in f32
            assert Fraction(float(y[b, 2 * j])) == d * (lo - 8)
            assert Fraction(float(y[b, 2 * j + 1])) == d * (hi - 8)


def test_dequant_q4_0_orders_are_a_permutation_of_each_other():
    blocks = synth.random_blocks(Q4_0, 32, seed=2)
    yc = o.dequantize(Q4_0, blocks).reshape(-1, 32)
    yg = o.dequantize(Q4_0_GGML, blocks).reshape(-1, 32)
    # ggml order (quantized.cu:862-866): y[j] <- low nibble of qs[j], y[j+16] <- high nibble
    assert np.array_equal(yc[:, 0::2], yg[:, :16])
    assert np.array_equal(yc[:, 1::2], yg[:, 16:])
    assert not np.array_equal(yc, yg)


def test_dequant_q8_0_exact():
    blocks = synth.random_blocks(Q8_0, 64, seed=3).view(synth.BLOCK_DTYPES[Q8_0]).copy()
    for i, s in enumerate(_special_scales()):
        blocks["d"][i] = s
    blocks["qs"][0][:4] = [-128, 127, 0, -1]
    y = o.dequantize(Q8_0, blocks).reshape(-1, 32)
    for b in range(len(blocks)):
        d = half_fraction(int(blocks["d"][b]))
        for i in range(32):
            assert Fraction(float(y[b, i])) == d * int(blocks["qs"][b][i])


def test_scale_min_k4_matches_masked_u16_reading():
    rng = np.random.default_rng(11)
    pats = [rng.integers(0, 256, 12, dtype=np.uint8) for _ in range(2000)]
    pats += [np.full(12, v, np.uint8) for v in (0, 0xFF, 0x3F, 0xC0, 0x0F, 0xF0, 0x40, 0x80)]
    # exhaustive over each byte that a j>=4 entry mixes: q[j+4] with q[j-4] and q[j]
    for j in range(4, 8):
        for a in range(0, 256, 5):
            for b in range(0, 256, 7):
                p = rng.integers(0, 256, 12, dtype=np.uint8)
                p[j + 4], p[j - 4], p[j] = a, b, (a * 3 + b) & 0xFF
                pats.append(p)
    for p in pats:
        sc, mn = k4_from_masked_u16(p)
        for j in range(8):
            assert o.get_scale_min_k4(j, p) == (sc[j], mn[j])
    # every 6-bit value is reachable in every slot
    seen = {(j, v) for p in pats[:2000] for j in range(8) for v in o.get_scale_min_k4(j, p)}
    assert all((j, 63) in seen and (j, 0) in seen for j in range(8))


def test_dequant_q4_k_is_one_rounding_of_the_exact_value():
    n = 24
    blocks = synth.random_blocks(Q4_K, n, seed=4).view(synth.BLOCK_DTYPES[Q4_K]).copy()
    sp = _special_scales()
    for i in range(len(sp)):
        blocks["d"][i] = sp[i]
        blocks["dmin"][i] = sp[(i * 3 + 1) % len(sp)]
    y = o.dequantize(Q4_K, blocks).reshape(n, 256)
    for b in range(n):
        d, dmin = half_fraction(int(blocks["d"][b])), half_fraction(int(blocks["dmin"][b]))
        sc, mn = k4_from_masked_u16(blocks["scales"][b])
        for e in range(256):
            t = e // 32
            exact = d * sc[t] * q4k_quant(blocks[b], e) - dmin * mn[t]
            assert y[b, e] == frac_to_f32(exact), (b, e)


def test_dequant_q6_k_exact():
    n = 24
    blocks = synth.random_blocks(Q6_K, n, seed=5).view(synth.BLOCK_DTYPES[Q6_K]).copy()
    for i, s in enumerate(_special_scales()):
        blocks["d"][i] = s
    blocks["scales"][0][:3] = [-128, 127, 0]
    y = o.dequantize(Q6_K, blocks).reshape(n, 256)
    for b in range(n):
        d = half_fraction(int(blocks["d"][b]))
        for e in range(256):
            exact = d * int(blocks["scales"][b][e // 16]) * q6_quant(blocks[b], e)
            assert Fraction(float(y[b, e])) == exact, (b, e)


def test_dequantize_rejects_unknown_format_and_ragged_bytes():
    assert o.lib().co_dequantize(77, None, 0, None) == -1
    with pytest.raises(AssertionError):
        o.dequantize(Q4_K, np.zeros(143, np.uint8))
    assert o.dequantize(Q4_K, np.zeros(0, np.uint8)).size == 0


# ---------------------------------------------------------------- activation quantizer

def _quantize_reference(x: np.ndarray):
    """float64 evaluation of quantized.cu:3546-3556 on one row-major [nb, 32] array."""
    x = x.astype(np.float32).reshape(-1, 32)
    amax = np.max(np.abs(x), axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)  # IEEE f32 division
    with np.errstate(divide="ignore", invalid="ignore"):
        v = (x / d[:, None]).astype(np.float32).astype(np.float64)  # f32 division, then exact widening
    q = np.where(amax[:, None] == 0, 0.0, np.trunc(v + np.copysign(0.5, v)))  # round half away from zero
    with np.errstate(over="ignore"):
        return q.astype(np.int8), d.astype(np.float16).view(np.uint16)


def test_quantize_q8_0_matches_float64_evaluation():
    rng = np.random.default_rng(21)
    x = rng.standard_normal((64, 256)).astype(np.float32)
    x[0, :32] = 0.0                       # all-zero block
    x[1, :32] = 1e-30                     # scale underflows fp16 to zero, quants still 127
    x[2, :32] = np.linspace(-3, 3, 32)    # ties: values at exactly +-amax
    x[3, :32] = np.float32(2.5) * np.arange(-16, 16)  # many exact .5 quotients
    x[4, :32] = 6e4                       # amax/127 fits fp16; large values
    x[5, :32] = 1e7                       # scale overflows fp16 range of normal numbers? (78740 -> inf)
    x[6, :32] = -0.0
    q, dbits = _quantize_reference(x)
    out = o.quantize_q8_0(x).view(synth.BLOCK_DTYPES[Q8_0])
    assert np.array_equal(out["qs"], q)
    assert np.array_equal(out["d"], dbits)
    # invariants
    nz = np.max(np.abs(x.reshape(-1, 32)), axis=1) > 0
    assert np.all(np.max(np.abs(out["qs"].astype(np.int32)), axis=1)[nz] == 127)
    assert np.all(out["qs"][~nz] == 0) and np.all(out["d"][~nz] == 0)
    assert out["qs"].min() >= -127


def test_quantize_q8_0_half_away_from_zero():
    # amax = 127 -> d = 1 exactly, so x/d = x and .5 values must round away from zero
    x = np.zeros(32, np.float32)
    x[:8] = [127, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5]
    out = o.quantize_q8_0(x).view(synth.BLOCK_DTYPES[Q8_0])
    assert list(out["qs"][0][:8]) == [127, 1, -1, 2, -2, 3, -3, 127]
    assert out["d"][0] == 0x3C00


def test_quantize_q8_0_shape_errors():
    assert o.lib().co_quantize_q8_0(None, 1, 33, None) == -1
    assert o.quantize_q8_0(np.zeros((0, 32), np.float32), 0, 32).size == 0


# ---------------------------------------------------------------- vec-dot / QMatMul

def _exact_dot(fmt: int, wrow: np.ndarray, xq: np.ndarray) -> Fraction:
    """Sum over the row of (exact weight value) * (exact dequantized activation)."""
    xb = xq.view(synth.BLOCK_DTYPES[Q8_0])
    xs = [half_fraction(int(b["d"])) for b in xb]
    wb = wrow.view(synth.BLOCK_DTYPES[fmt])
    total = Fraction(0)
    for bi, blk in enumerate(wb):
        if fmt in (Q4_0, Q4_0_GGML):
            d = half_fraction(int(blk["d"]))
            for j in range(16):
                lo, hi = int(blk["qs"][j]) & 15, int(blk["qs"][j]) >> 4
                i_lo, i_hi = (2 * j, 2 * j + 1) if fmt == Q4_0 else (j, j + 16)
                total += d * (lo - 8) * xs[bi] * int(xb[bi]["qs"][i_lo])
                total += d * (hi - 8) * xs[bi] * int(xb[bi]["qs"][i_hi])
        elif fmt == Q8_0:
            d = half_fraction(int(blk["d"]))
            total += d * xs[bi] * sum(int(a) * int(b) for a, b in zip(blk["qs"], xb[bi]["qs"]))
        elif fmt == Q4_K:
            d, dmin = half_fraction(int(blk["d"])), half_fraction(int(blk["dmin"]))
            sc, mn = k4_from_masked_u16(blk["scales"])
            for e in range(256):
                t = e // 32
                w = d * sc[t] * q4k_quant(blk, e) - dmin * mn[t]
                total += w * xs[8 * bi + t] * int(xb[8 * bi + t]["qs"][e % 32])
        elif fmt == Q6_K:
            d = half_fraction(int(blk["d"]))
            for e in range(256):
                w = d * int(blk["scales"][e // 16]) * q6_quant(blk, e)
                total += w * xs[8 * bi + e // 32] * int(xb[8 * bi + e // 32]["qs"][e % 32])
    return total


@pytest.mark.parametrize("fmt", [Q4_0, Q4_0_GGML, Q8_0, Q4_K, Q6_K])
def test_vec_dot_equals_exact_sum_of_dequantized_products(fmt):
    k = 512
    rows = 6
    w = synth.random_weight(fmt, rows, k, seed=100 + fmt)
    x = synth.random_activations(1, k, seed=200 + fmt)
    xq = o.quantize_q8_0(x)
    rb = synth.weight_nbytes(fmt, 1, k)
    for r in range(rows):
        wrow = w[r * rb:(r + 1) * rb]
        got = o.vec_dot_q8_0(fmt, wrow, xq, k)
        exact = _exact_dot(fmt, wrow, xq)
        # f32 accumulation of <= 16 block terms: error far below 1e-5 of the absolute mass
        mass = float(sum(abs(v) for v in o.dequantize(fmt, wrow))) * 5.0
        assert abs(Fraction(got) - exact) <= Fraction(1e-6) * Fraction(mass) + Fraction(1e-30), (fmt, r)


@pytest.mark.parametrize("fmt", [Q4_0, Q8_0, Q4_K, Q6_K])
def test_qmatmul_equals_naive_f32_matmul_on_dequantized_operands(fmt):
    # same mathematics as candy's literal CPU composition (dequantize, then conv.go:373-389)
    # once the activations have gone through Q8_0; only f32 rounding order differs
    rows, k, m = 48, 1024, 3
    w = synth.random_weight(fmt, rows, k, seed=300 + fmt)
    x = synth.random_activations(m, k, seed=400 + fmt)
    xdq = o.dequantize(Q8_0, o.quantize_q8_0(x)).reshape(m, k)
    a = o.qmatmul(fmt, w, rows, k, x)
    b = o.matmul_dequant_f32(fmt, w, rows, k, xdq)
    assert a.shape == b.shape == (m, rows)
    assert np.max(np.abs(a - b)) <= 2e-5 * np.max(np.abs(b))
    # and the un-quantized activations give the informational distance (about 5e-3), not parity
    c = o.matmul_dequant_f32(fmt, w, rows, k, x)
    assert 1e-5 < np.max(np.abs(a - c)) / np.max(np.abs(c)) < 5e-2


def test_matmul_dequant_equals_float64_matmul():
    rows, k, m = 16, 512, 2
    w = synth.random_weight(Q4_K, rows, k, seed=9)
    x = synth.random_activations(m, k, seed=10)
    wf = o.dequantize(Q4_K, w).reshape(rows, k).astype(np.float64)
    want = x.astype(np.float64) @ wf.T
    got = o.matmul_dequant_f32(Q4_K, w, rows, k, x)
    assert np.max(np.abs(got - want)) <= 1e-5 * np.max(np.abs(want))


def test_qmatmul_linearity_in_weight_scale():
    # doubling every fp16 super-block scale doubles the result exactly (power-of-two scaling)
    rows, k = 8, 512
    w = synth.random_weight(Q4_K, rows, k, seed=12).view(synth.BLOCK_DTYPES[Q4_K]).copy()
    w["d"] = (w["d"].view(np.float16) * np.float16(1)).view(np.uint16)
    x = synth.random_activations(1, k, seed=13)
    y1 = o.qmatmul(Q4_K, w, rows, k, x)
    w2 = w.copy()
    w2["d"] = (w["d"].view(np.float16) * np.float16(2)).view(np.uint16)
    w2["dmin"] = (w["dmin"].view(np.float16) * np.float16(2)).view(np.uint16)
    y2 = o.qmatmul(Q4_K, w2, rows, k, x)
    assert np.array_equal(y2, 2 * y1)
