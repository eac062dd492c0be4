"""Weight quantizers from f32 on the device against the CPU oracle: the blocks must be bit for bit equal
(the search of the K formats is a chain of f32 comparisons, so one differently rounded operation shows)."""
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


def matrix(seed: int, rows: int, cols: int) -> np.ndarray:
    """Rows of different character, with an all-zero block, a constant block and a single spike mixed in."""
    rng = np.random.default_rng(seed)
    x = np.empty((rows, cols), np.float32)
    for r in range(rows):
        kind = r % 5
        if kind == 0:
            x[r] = rng.standard_normal(cols) * 0.02
        elif kind == 1:
            x[r] = rng.uniform(-1, 1, cols)
        elif kind == 2:
            x[r] = rng.standard_t(2, cols) * 0.1
        elif kind == 3:
            x[r] = np.abs(rng.standard_normal(cols)) + 0.5
        else:
            x[r] = rng.standard_normal(cols) * 1e-6
    x[0, :256] = 0.0
    if rows > 1:
        x[1, :256] = 0.25
    if rows > 2:
        x[2, :256] = 0.0
        x[2, 131] = -7.5
    return x


@pytest.mark.parametrize("fmt", FORMATS, ids=lambda f: synth.FORMAT_NAMES[f])
@pytest.mark.parametrize("rows,cols", [(1, 256), (11, 1024), (3, 4096), (130, 512)])
def test_blocks_equal_the_oracle(dev, fmt, rows, cols):
    x = matrix(rows * 1000 + cols + fmt, rows, cols)
    got = dev.quantize(fmt, x)
    want = o.quantize(fmt, x)
    assert got.size == synth.weight_nbytes(fmt, rows, cols)
    if not np.array_equal(got, want):
        bs = synth.BLOCK_BYTES[fmt]
        bad = np.flatnonzero(np.any(got.reshape(-1, bs) != want.reshape(-1, bs), axis=1))
        raise AssertionError(f"{len(bad)} of {got.size // bs} blocks differ, first {bad[:5]}")


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q4_0], ids=lambda f: synth.FORMAT_NAMES[f])
def test_quantized_weight_feeds_the_matmul(dev, fmt):
    # quantize(N(0, 0.02)) on the device, contract without leaving it; the CPU does the same with its own blocks
    rng = np.random.default_rng(8)
    rows, cols = 96, 1024
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    x = synth.random_activations(3, cols, seed=9)
    q = hip.QTensor.quantize(dev, fmt, w)
    got = dev.qmatmul(q, x)
    want = o.qmatmul(fmt, o.quantize(fmt, w), rows, cols, x)
    assert np.max(np.abs(got - want)) <= 1e-3 * np.max(np.abs(want))
    # and the quantized weight is the matrix it came from, to the format's accuracy
    full = x.astype(np.float64) @ w.astype(np.float64).T
    bound = {synth.Q4_K: 0.12, synth.Q6_K: 0.04, synth.Q4_0: 0.16}[fmt]
    assert np.sqrt(np.mean((got - full) ** 2) / np.mean(full ** 2)) < bound
    q.free()


def test_weight_quantized_on_the_device_takes_the_same_kernels_as_an_uploaded_one(dev):
    # a Q6_K row's last 16-byte load in the int8 tile kernel starts inside the last block and runs past it, so the
    # kernel takes only buffers known to have room there: uploads (padded by the library) and wrapped buffers whose
    # stated size says so, which is how QTensor.quantize wraps its blocks.  Same kernel, same bits at 8 and 40 rows.
    rng = np.random.default_rng(18)
    rows, cols = 256, 2048
    w = (rng.standard_normal((rows, cols)) * 0.02).astype(np.float32)
    q_dev = hip.QTensor.quantize(dev, synth.Q6_K, w)
    q_up = dev.qtensor(synth.Q6_K, rows, cols, dev.quantize(synth.Q6_K, w))
    for m in (8, 40):
        x = synth.random_activations(m, cols, seed=m)
        a, b = dev.qmatmul(q_dev, x), dev.qmatmul(q_up, x)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), m
    # a wrapped buffer without spare bytes still works (other tiles, fp16 operands from 16 rows on)
    blocks = dev.from_numpy(dev.quantize(synth.Q6_K, w))
    h = hip.c_void_p()
    hip._check(hip.lib().candy_hip_qtensor_wrap(dev.handle, synth.Q6_K, rows, cols, blocks.ptr, blocks.nbytes, hip.byref(h)))
    tight = hip.QTensor.__new__(hip.QTensor)
    tight.dev, tight.fmt, tight.rows, tight.cols, tight.nbytes, tight.handle, tight._blocks = dev, synth.Q6_K, rows, cols, blocks.nbytes, h.value, blocks
    x = synth.random_activations(40, cols, seed=40)
    want = dev.qmatmul(q_up, x)
    got = dev.qmatmul(tight, x)
    assert np.max(np.abs(got - want)) <= 1e-3 * np.max(np.abs(want))
    with pytest.raises(hip.CandyHipError, match="need"):   # a buffer smaller than the blocks is refused
        hip._check(hip.lib().candy_hip_qtensor_wrap(dev.handle, synth.Q6_K, rows, cols, blocks.ptr, blocks.nbytes - 1, hip.byref(h)))
    for t in (q_dev, q_up, tight):
        t.free()


def test_quantize_errors_and_empty(dev):
    assert dev.quantize(synth.Q4_K, np.zeros((0, 256), np.float32)).size == 0
    with pytest.raises(hip.CandyHipError, match="multiple of the block"):
        dev.quantize(synth.Q4_K, np.zeros((2, 128), np.float32))
    with pytest.raises(hip.CandyHipError, match="unknown block format"):
        dev.quantize(77, np.zeros((2, 256), np.float32))
