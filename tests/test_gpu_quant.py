"""GPU parity, bit-exact part: dequantize (4 formats + both Q4_0 orders) and the Q8_0
activation quantizer against the CPU oracle on identical seeded bytes."""
import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import oracle as o

pytestmark = pytest.mark.gpu

FORMATS = [synth.Q4_0, synth.Q4_0_GGML, synth.Q8_0, synth.Q4_K, synth.Q6_K]


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("n_blocks", [1, 7, 64, 1000])
def test_dequantize_bit_exact(dev, fmt, n_blocks):
    blocks = synth.random_blocks(fmt, n_blocks, seed=1000 + fmt + n_blocks)
    dt = synth.BLOCK_DTYPES[fmt]
    b = blocks.view(dt).copy()
    # scale edge cases: zero, subnormal, max normal, negative
    for i, s in enumerate([0x0000, 0x0001, 0x03FF, 0x7BFF, 0xFBFF, 0x8000][: min(6, n_blocks)]):
        b["d"][i] = s
    got = dev.dequantize_blocks(fmt, b)
    want = o.dequantize(fmt, b)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q8_0, synth.Q4_0])
def test_dequantize_full_weight_matrix(dev, fmt):
    rows, cols = 512, 4096
    w = synth.random_weight(fmt, rows, cols, seed=7 + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.dequantize(q)
    want = o.dequantize(fmt, w).reshape(rows, cols)
    assert np.array_equal(_bits(got), _bits(want))


def test_dequantize_empty(dev):
    assert dev.dequantize_blocks(synth.Q4_K, np.zeros(0, np.uint8)).size == 0


@pytest.mark.parametrize("shape", [(1, 32), (1, 4096), (3, 11008), (16, 4096), (512, 4096)])
def test_quantize_q8_0_bit_exact(dev, shape):
    x = synth.random_activations(shape[0], shape[1], seed=shape[0] * 131 + shape[1])
    got = dev.quantize_q8_0(x)
    want = o.quantize_q8_0(x)
    assert np.array_equal(got, want)


def test_quantize_q8_0_edge_blocks(dev):
    x = synth.random_activations(8, 256, seed=5)
    x[0, :32] = 0.0
    x[0, 32:64] = -0.0
    x[1, :32] = 1e-30                                  # scale underflows fp16
    x[2, :32] = np.float32(2.5) * np.arange(-16, 16)   # exact .5 quotients round away from zero
    x[3, :8] = [127, 0.5, -0.5, 1.5, -1.5, 2.5, -2.5, 126.5]
    x[3, 8:32] = 0
    x[4, :32] = 6e4
    x[5, :32] = 1e7                                    # scale overflows fp16 to inf
    x[6, :32] = np.linspace(-3, 3, 32)
    x[7, :32] = 1e-41                                  # f32 subnormal inputs
    got = dev.quantize_q8_0(x)
    want = o.quantize_q8_0(x)
    assert np.array_equal(got, want)
    blk = got.view(synth.BLOCK_DTYPES[synth.Q8_0])
    assert list(blk["qs"][3 * 8][:8]) == [127, 1, -1, 2, -2, 3, -3, 127]


def test_quantize_q8_0_quotients_next_to_half_integers(dev):
    # The device forms x / d as x * (1 / d) and divides only where that product is within a few ulp of a
    # half-integer (where the two could round to different levels).  Blocks built to sit on that edge: one element
    # fixes the scale, the others are the f32 numbers around d * (k + 0.5) for every k, for many scales.
    rng = np.random.default_rng(77)
    rows = []
    for trial in range(400):
        amax = np.float32(rng.uniform(0.01, 100.0) * 10.0 ** rng.integers(-3, 3))
        d = np.float32(amax / np.float32(127.0))
        ks = rng.integers(0, 127, 31)
        halves = (d.astype(np.float64) * (ks + 0.5)).astype(np.float32)
        steps = rng.integers(-3, 4, 31)
        xs = halves.copy()
        for i, st in enumerate(steps):  # walk a few representable numbers to either side of the midpoint
            for _ in range(abs(int(st))):
                xs[i] = np.nextafter(xs[i], np.float32(np.inf if st > 0 else -np.inf))
        xs *= rng.choice(np.array([-1.0, 1.0], np.float32), 31)
        rows.append(np.concatenate([[amax if trial % 2 else -amax], xs]).astype(np.float32))
    x = np.stack(rows)
    got, want = dev.quantize_q8_0(x), o.quantize_q8_0(x)
    assert np.array_equal(got, want)
    levels = want.view(synth.BLOCK_DTYPES[synth.Q8_0])["qs"]
    assert np.abs(levels).max() == 127 and len(np.unique(np.abs(levels))) > 100


def test_quantize_q8_0_errors(dev):
    with pytest.raises(hip.CandyHipError, match="multiple of the block size"):
        dev.quantize_q8_0(np.zeros((2, 48), np.float32))


def test_quantize_then_dequantize_round_trip_property(dev):
    # size-independent property at full size: |x - dq(q(x))| <= d/2 per element (+ fp16 rounding of d)
    x = synth.random_activations(512, 4096, seed=99)
    blocks = dev.quantize_q8_0(x)
    y = dev.dequantize_blocks(synth.Q8_0, blocks).reshape(x.shape)
    d = blocks.view(synth.BLOCK_DTYPES[synth.Q8_0])["d"].view(np.float16).astype(np.float32)
    bound = np.repeat(d, 32).reshape(x.shape) * (0.5 + 127 * 2.0 ** -11) + 1e-12
    assert np.all(np.abs(x - y) <= bound)


def test_qindex_select_matches_dequantized_rows(dev):
    rows, cols = 300, 1024
    for fmt in (synth.Q8_0, synth.Q4_K, synth.Q6_K):
        w = synth.random_weight(fmt, rows, cols, seed=31 + fmt)
        q = dev.qtensor(fmt, rows, cols, w)
        ids = np.array([5, 0, 299, 5, 17], np.int64)
        got = dev.qindex_select(q, ids)
        want = o.dequantize(fmt, w).reshape(rows, cols)[ids]
        assert np.array_equal(_bits(got), _bits(want))
