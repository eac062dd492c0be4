"""GPU parity of the reference's other dequantize outputs (fp16, float64), bit for bit, and of its f32-activation
matvec (dequantize_mul_mat_vec) against candy's CPU path (dequantize, then the naive f32 MatMul)."""
import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import oracle as o

pytestmark = pytest.mark.gpu

ALL = [synth.Q4_0, synth.Q4_0_GGML, synth.Q8_0, synth.Q4_K, synth.Q6_K, synth.Q4_1, synth.Q4_1_GGML, synth.Q5_0, synth.Q5_1,
       synth.Q2_K, synth.Q3_K, synth.Q5_K, synth.Q8_K]
name = lambda f: synth.FORMAT_NAMES[f]  # noqa: E731
SPECIAL = [0x0000, 0x0001, 0x03FF, 0x7BFF, 0xFBFF, 0x8000]


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def edge_blocks(fmt, n_blocks, seed):
    dt = synth.BLOCK_DTYPES[fmt]
    b = synth.random_blocks(fmt, n_blocks, seed=seed).view(dt).copy()
    if fmt != synth.Q8_K:  # scale edge cases: zero, subnormal, max normal, negative
        for i, s in enumerate(SPECIAL[: min(6, n_blocks)]):
            b["d"][i] = s
            for other in ("m", "dmin"):
                if other in dt.names:
                    b[other][i] = SPECIAL[(i + 2) % 6]
    return b


@pytest.mark.parametrize("fmt", ALL, ids=name)
@pytest.mark.parametrize("n_blocks", [1, 7, 1000])
def test_dequantize_f16_bit_exact(dev, fmt, n_blocks):
    # dequantize_block_*_f16 (kernels.go:486-505): the f32 value, rounded to nearest even on the store; values past
    # fp16's range become infinities on both sides (max-normal scales are among the cases)
    b = edge_blocks(fmt, n_blocks, 3000 + fmt + n_blocks)
    got = dev.dequantize_blocks_as(fmt, b, np.float16)
    with np.errstate(over="ignore"):
        want = o.dequantize_f16(fmt, b)
    assert got.dtype == np.float16 and np.array_equal(got.view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q8_0])
def test_dequantize_f16_weight_matrix(dev, fmt):
    rows, cols = 256, 4096
    w = synth.random_weight(fmt, rows, cols, seed=11 + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.dequantize_f16(q)
    assert np.array_equal(got.view(np.uint16), o.dequantize_f16(fmt, w).reshape(rows, cols).view(np.uint16))
    # and it is the f32 output of the device rounded once
    assert np.array_equal(got.view(np.uint16), dev.dequantize(q).astype(np.float16).view(np.uint16))


@pytest.mark.parametrize("fmt", [synth.Q4_0, synth.Q4_1, synth.Q8_0], ids=name)
@pytest.mark.parametrize("n_blocks", [1, 7, 1000])
def test_dequantize_f64_bit_exact(dev, fmt, n_blocks):
    # DequantizeBlockQ4_0F64 / Q4_1F64 / Q8_0F64 (quantized.go:96-104, 119-128, 139-144)
    b = edge_blocks(fmt, n_blocks, 4000 + fmt + n_blocks)
    got = dev.dequantize_blocks_as(fmt, b, np.float64)
    want = o.dequantize_f64(fmt, b)
    assert got.dtype == np.float64 and np.array_equal(got.view(np.uint64), want.view(np.uint64))


NONFINITE = [0x7C00, 0xFC00, 0x7E00, 0x7D00, 0xFE01, 0x7FFF]  # +inf, -inf, quiet NaN, signalling NaN, NaNs with payload


def nonfinite_blocks(fmt, seed):
    """Random blocks whose fp16 scale fields run through infinities and NaNs, one field at a time and together."""
    dt = synth.BLOCK_DTYPES[fmt]
    fields = [f for f in ("d", "m", "dmin") if f in dt.names]
    n = len(NONFINITE) * (len(fields) + 1) + 2
    b = synth.random_blocks(fmt, n, seed=seed).view(dt).copy()
    if fmt == synth.Q8_K:  # an f32 scale
        b["d"][: len(NONFINITE)] = np.array([0x7F800000, 0xFF800000, 0x7FC00000, 0x7FA00000, 0xFFC00001, 0x7FFFFFFF],
                                            np.uint32).view(np.float32)
        return b
    i = 0
    for f in fields:
        for s in NONFINITE:
            b[f][i] = s
            i += 1
    for k, s in enumerate(NONFINITE):  # every scale field of the block non-finite, with different patterns
        for j, f in enumerate(fields):
            b[f][i] = NONFINITE[(k + j) % len(NONFINITE)]
        i += 1
    return b


@pytest.mark.parametrize("fmt", ALL, ids=name)
def test_dequantize_with_infinite_and_nan_scales(dev, fmt):
    # fp16ToFloat32 (quantized.go:149-173) widens an infinite scale to an infinity and a NaN scale to a NaN that
    # keeps its payload (:156); the products then follow IEEE: inf * 0 and anything with a NaN are NaNs, the rest
    # signed infinities.  Which NaN comes out (sign, payload, quiet bit) is not fixed by the arithmetic - the CPU's
    # default NaN has the sign bit set, the GPU's does not, and each keeps the payload of a different operand - so
    # NaN positions are compared as NaNs and every other element bit for bit, in each output type.
    b = nonfinite_blocks(fmt, 5000 + fmt)
    outputs = [(np.float32, np.uint32, o.dequantize), (np.float16, np.uint16, o.dequantize_f16)]
    if fmt in (synth.Q4_0, synth.Q4_1, synth.Q8_0):
        outputs.append((np.float64, np.uint64, o.dequantize_f64))
    for dtype, bits, ref in outputs:
        with np.errstate(all="ignore"):
            want = np.asarray(ref(fmt, b))
        got = dev.dequantize_blocks(fmt, b) if dtype is np.float32 else dev.dequantize_blocks_as(fmt, b, dtype)
        got = np.asarray(got).reshape(want.shape)
        nan = np.isnan(want)
        # the cases are really there (the ggml-order Q4_0 is d * q + (-8 d), quantized.cu:857-866: inf - inf, all NaNs)
        assert nan.any() and (fmt == synth.Q4_0_GGML or np.isinf(want).any()), name(fmt)
        assert np.array_equal(np.isnan(got), nan), (name(fmt), dtype)
        assert np.array_equal(got.view(bits)[~nan], want.view(bits)[~nan]), (name(fmt), dtype)


def test_dequantize_outputs_errors_and_empty(dev):
    assert dev.dequantize_blocks_as(synth.Q4_K, np.zeros(0, np.uint8), np.float16).size == 0
    assert dev.dequantize_blocks_as(synth.Q8_0, np.zeros(0, np.uint8), np.float64).size == 0
    with pytest.raises(hip.CandyHipError, match="Q4_0, Q4_1 and Q8_0 only"):   # the CPU kernels have no other twins
        dev.dequantize_blocks_as(synth.Q4_K, synth.random_blocks(synth.Q4_K, 2, seed=1), np.float64)
    with pytest.raises(hip.CandyHipError, match="unknown quantized format"):
        dev.dequantize_blocks_as(99, np.zeros(18, np.uint8), np.float16)


@pytest.mark.parametrize("fmt", [f for f in ALL if f != synth.Q8_K], ids=name)
@pytest.mark.parametrize("rows,cols", [(64, 256), (37, 512), (130, 4096), (9, 11008)])
def test_dmmv_matches_dequantize_then_matmul(dev, fmt, rows, cols):
    # dequantize_mul_mat_vec (quantized.cu:1251-1345, :1550-1693, :1810-1911): f32 activations, no Q8_0 rounding.
    # Same products as Dequantize + naive MatMul (cpu/storage.go:893-910 -> conv.go:373-389), summed in another
    # order: 2e-5 of the largest output (observed ~1e-6)
    w = synth.random_weight(fmt, rows, cols, seed=rows + cols + fmt)
    x = synth.random_activations(1, cols, seed=cols + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.dmmv(q, x)
    want = o.matmul_dequant_f32(fmt, w, rows, cols, x).reshape(-1)
    assert got.shape == (rows,)
    assert float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want))) <= 2e-5
    # against the exact sum (float64 of the same dequantized weights): no further from it than the CPU loop is, up
    # to the spacing of f32 sums of this length
    wd = o.dequantize(fmt, w).reshape(rows, cols).astype(np.float64)
    exact = wd @ x.reshape(-1).astype(np.float64)
    scale = np.max(np.abs(exact))
    assert np.max(np.abs(got - exact)) / scale <= max(2 * np.max(np.abs(want - exact)) / scale, 1e-6)
    q.free()


def test_dmmv_full_shape_and_linearity(dev):
    rows, cols = 4096, 11008
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=21)
    x = synth.random_activations(1, cols, seed=22)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    got = dev.dmmv(q, x)
    sub = np.arange(0, rows, 64)
    rb = synth.weight_nbytes(synth.Q4_K, 1, cols)
    want = o.matmul_dequant_f32(synth.Q4_K, w.reshape(rows, rb)[sub].reshape(-1), len(sub), cols, x).reshape(-1)
    assert float(np.max(np.abs(got[sub] - want)) / np.max(np.abs(want))) <= 2e-5
    assert np.array_equal(dev.dmmv(q, 2 * x), 2 * got)     # exact: no quantizer between x and the sum
    # and closer to the exact product than the quantized-activation matvec is
    wd = o.dequantize(synth.Q4_K, w.reshape(rows, rb)[sub].reshape(-1)).reshape(len(sub), cols).astype(np.float64)
    exact = wd @ x.reshape(-1).astype(np.float64)
    assert np.max(np.abs(got[sub] - exact)) < np.max(np.abs(dev.qmatmul(q, x)[0, sub] - exact))
    with pytest.raises(hip.CandyHipError, match="no f32-activation matvec"):
        w8 = synth.random_weight(synth.Q8_K, 4, 256, seed=1)
        dev.dmmv(dev.qtensor(synth.Q8_K, 4, 256, w8), np.zeros(256, np.float32))
