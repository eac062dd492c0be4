"""The reference's other block formats on the device (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K) against the
oracle: dequantize and row gather bit for bit, QMatMul within 1e-3 (max-norm) at every batch size."""
import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import oracle as o

pytestmark = pytest.mark.gpu

NEW = [synth.Q4_1, synth.Q4_1_GGML, synth.Q5_0, synth.Q5_1, synth.Q2_K, synth.Q3_K, synth.Q5_K, synth.Q8_K]
MATMUL = [f for f in NEW if f != synth.Q8_K]
name = lambda f: synth.FORMAT_NAMES[f]  # noqa: E731
TOL = 1e-3


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def rel_err(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / np.max(np.abs(want)))


@pytest.mark.parametrize("fmt", NEW, ids=name)
@pytest.mark.parametrize("n_blocks", [1, 7, 64, 1000])
def test_dequantize_bit_exact(dev, fmt, n_blocks):
    dt = synth.BLOCK_DTYPES[fmt]
    b = synth.random_blocks(fmt, n_blocks, seed=2000 + fmt + n_blocks).view(dt).copy()
    if fmt != synth.Q8_K:  # scale edge cases: zero, subnormal, max normal, negative
        special = [0x0000, 0x0001, 0x03FF, 0x7BFF, 0xFBFF, 0x8000]
        for i, s in enumerate(special[: min(6, n_blocks)]):
            b["d"][i] = s
            for other in ("m", "dmin"):
                if other in dt.names:
                    b[other][i] = special[(i + 2) % 6]
    got = dev.dequantize_blocks(fmt, b)
    want = o.dequantize(fmt, b)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("fmt", NEW, ids=name)
def test_weight_matrix_dequantize_and_row_gather(dev, fmt):
    rows, cols = 300, 1024
    w = synth.random_weight(fmt, rows, cols, seed=7 + fmt, scale=synth.unit_scale(fmt))
    q = dev.qtensor(fmt, rows, cols, w)
    want = o.dequantize(fmt, w).reshape(rows, cols)
    assert np.array_equal(_bits(dev.dequantize(q)), _bits(want))
    ids = np.array([5, 0, 299, 5, 17], np.int64)
    assert np.array_equal(_bits(dev.qindex_select(q, ids)), _bits(want[ids]))


@pytest.mark.parametrize("fmt", MATMUL, ids=name)
@pytest.mark.parametrize("rows,cols", [(64, 256), (37, 512), (256, 4096), (130, 11008), (8, 14336)])
def test_matvec_matches_oracle(dev, fmt, rows, cols):
    w = synth.random_weight(fmt, rows, cols, seed=rows * 7 + cols + fmt, scale=synth.unit_scale(fmt))
    x = synth.random_activations(1, cols, seed=cols + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (1, rows)
    assert rel_err(got, want) <= TOL
    assert rel_err(got, want) <= 2e-5  # integer dot products, f32 only in the combination: a dropped group would show


@pytest.mark.parametrize("fmt", MATMUL, ids=name)
@pytest.mark.parametrize("m", [2, 5, 15, 16, 40, 300])
def test_batched_matmul_matches_oracle(dev, fmt, m):
    # 2..15 rows: the small-batch kernel (integer dots); from 16 rows: fp16 matrix-core tiles fed by the format's
    # dequantize (fp16 operand rounding, about 3e-4)
    rows, cols = 96, 2048
    w = synth.random_weight(fmt, rows, cols, seed=m + fmt, scale=synth.unit_scale(fmt))
    x = synth.random_activations(m, cols, seed=3 * m + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (m, rows)
    assert rel_err(got, want) <= (2e-5 if m < 16 else TOL)


@pytest.mark.parametrize("fmt", MATMUL, ids=name)
def test_tile_kernel_on_ragged_shapes(dev, fmt):
    # rows off the tile height, a contraction length with an odd number of 64-value steps (small-batch kernel in slices)
    for rows, cols, m in ((37, 512, 33), (130, 2304 if synth.BLOCK_ELEMS[fmt] == 256 else 2080, 17)):
        w = synth.random_weight(fmt, rows, cols, seed=rows + fmt, scale=synth.unit_scale(fmt))
        x = synth.random_activations(m, cols, seed=cols + fmt)
        got = dev.qmatmul(dev.qtensor(fmt, rows, cols, w), x)
        assert rel_err(got, o.qmatmul(fmt, w, rows, cols, x)) <= TOL


def test_q8_k_weights_only_dequantize(dev):
    w = synth.random_weight(synth.Q8_K, 4, 256, seed=1)
    q = dev.qtensor(synth.Q8_K, 4, 256, w)
    with pytest.raises(hip.CandyHipError, match="only dequantize"):
        dev.qmatmul(q, synth.random_activations(1, 256, seed=2))
