"""GPU parity of QMatMul against the CPU oracle: max_n |gpu - ref| / max_n |ref| <= 1e-3
(the f32 accumulation order differs; integer block dots are exact on both sides)."""
import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import oracle as o

pytestmark = pytest.mark.gpu

TOL = 1e-3  # the stated bar; observed distances are ~1e-6
FORMATS = [synth.Q4_0, synth.Q4_0_GGML, synth.Q8_0, synth.Q4_K, synth.Q6_K]


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def rel_err(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / np.max(np.abs(want)))


@pytest.mark.parametrize("fmt", FORMATS)
@pytest.mark.parametrize("rows,cols", [(64, 256), (37, 512), (256, 4096), (130, 11008), (8, 14336)])
def test_matvec_matches_oracle(dev, fmt, rows, cols):
    w = synth.random_weight(fmt, rows, cols, seed=rows * 7 + cols + fmt)
    x = synth.random_activations(1, cols, seed=cols + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (1, rows)
    assert rel_err(got, want) <= TOL
    assert rel_err(got, want) <= 2e-5  # much tighter in practice; catches a dropped block or scale


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q8_0, synth.Q6_K, synth.Q4_0])
@pytest.mark.parametrize("m", [2, 3, 5, 8, 15])
def test_small_batch_matches_oracle(dev, fmt, m):
    rows, cols = 96, 4096
    w = synth.random_weight(fmt, rows, cols, seed=m + fmt)
    x = synth.random_activations(m, cols, seed=m * 3 + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (m, rows)
    assert rel_err(got, want) <= 2e-5


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML, synth.Q6_K])
@pytest.mark.parametrize("rows,cols", [(50, 11008), (4099, 1280), (600, 6144), (40, 15360)])
def test_small_batch_one_pass_per_eight_rows(dev, monkeypatch, fmt, rows, cols):
    # 3 .. 15 activation rows against long or many weight rows: one workgroup per CU holds up to eight quantized
    # rows in LDS and walks the weight rows (Q6_K: the looping kernel), or the int8 tile kernel takes the batch as
    # one 16-row tile.  The vector kernels add a lane's units in the same order as the looping kernel: same bits;
    # the tile kernel differs by f32 summation order only.  Row counts off the 16-row groups and more groups than
    # CUs (4099 rows) are in, and the longest row whose eight images still fit LDS (15360: 158 KB).
    w = synth.random_weight(fmt, rows, cols, seed=rows + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    for m in (3, 4, 5, 7, 8, 9, 13, 15):
        x = synth.random_activations(m, cols, seed=m * 5 + fmt)
        got = dev.qmatmul(q, x)
        assert got.shape == (m, rows)
        if m in (3, 8, 15):
            assert rel_err(got, o.qmatmul(fmt, w, rows, cols, x)) <= 2e-5, m
        try:
            dev.set_option("matvec.small_batch_kernel", 0)
            dev.set_option("mmq.i8_min_m", 99)
            old = dev.qmatmul(q, x)
            dev.set_option("mmq.i8_min_m", 2)  # tiles wherever they apply (Q4_K, Q6_K)
            tiles = dev.qmatmul(q, x)
            dev.set_option("matvec.small_batch_kernel", 1)
            dev.set_option("mmq.i8_min_m", 99)
            vector = dev.qmatmul(q, x)
        finally:
            dev.set_option("matvec.small_batch_kernel", 1)
            dev.set_option("mmq.i8_min_m", 0)
        assert np.array_equal(vector.view(np.uint32), old.view(np.uint32)), m
        assert rel_err(tiles, old) <= 2e-6, m
        assert rel_err(got, old) <= 2e-6, m


@pytest.mark.parametrize("rows,cols", [(4096, 256), (4100, 512), (11008, 4096), (4096, 11008), (4096, 8192),
                                       (4096, 14336), (12288, 1024), (9000, 2048)])
def test_two_rows_even_split_kernel(dev, rows, cols):
    # two activation rows against a Q4_K weight with 16 .. 48 rows per CU: the weight rows dealt evenly to two
    # workgroups per CU, one to three rows per wavefront, one to four rounds of units per row, row counts that do not
    # divide by the grid.  Same additions in the same order as the looping kernel: same bits.
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=rows + cols)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    sub = np.unique(np.concatenate([np.arange(0, rows, 97), np.arange(rows - 40, rows)]))
    wsub = w.reshape(rows, -1)[sub].reshape(-1)
    x = synth.random_activations(2, cols, seed=22 + cols)
    got = dev.qmatmul(q, x)
    try:
        dev.set_option("matvec.even_two_rows", 0)
        old = dev.qmatmul(q, x)
    finally:
        dev.set_option("matvec.even_two_rows", 1)
    assert np.array_equal(got.view(np.uint32), old.view(np.uint32))
    assert rel_err(got[:, sub], o.qmatmul(synth.Q4_K, wsub, len(sub), cols, x)) <= 2e-5


@pytest.mark.parametrize("fmt", [synth.Q8_0, synth.Q4_0, synth.Q5_1])
def test_five_to_eight_rows_on_a_big_weight_take_the_tile_kernel(dev, fmt):
    # 32-value formats, weights of 40 M values and more: 5 .. 8 rows run on the int8 tile kernel (integer-exact, like
    # the vector kernels they replace there: the two differ by f32 summation order only)
    rows, cols = 4096, 11008
    w = synth.random_weight(fmt, rows, cols, seed=fmt + 50)
    q = dev.qtensor(fmt, rows, cols, w)
    sub = np.arange(3, rows, 61)
    wsub = w.reshape(rows, -1)[sub].reshape(-1)
    for m in (5, 8):
        x = synth.random_activations(m, cols, seed=m + fmt)
        got = dev.qmatmul(q, x)
        assert rel_err(got[:, sub], o.qmatmul(fmt, wsub, len(sub), cols, x)) <= 2e-5, m
        try:
            dev.set_option("mmq.i8_min_m", 99)  # the vector kernels
            vector = dev.qmatmul(q, x)
        finally:
            dev.set_option("mmq.i8_min_m", 0)
        assert rel_err(got, vector) <= 2e-6, m
        assert not np.array_equal(got, vector), m  # another kernel did run


@pytest.mark.parametrize("fmt", [synth.Q6_K, synth.Q5_K])
def test_three_and_four_rows_on_long_weight_rows_take_the_tile_kernel(dev, fmt):
    # Q6_K / Q5_K with weight rows so long that the looping kernel holds one or two activation rows per launch:
    # 3 and 4 rows run as one 16-row int8 tile; on 4096-long weight rows the vector kernel keeps them
    for rows, cols, tiles in ((4096, 14336, True), (1024, 4096, False)):
        w = synth.random_weight(fmt, rows, cols, seed=fmt + 70)
        q = dev.qtensor(fmt, rows, cols, w)
        sub = np.arange(5, rows, 67)
        wsub = w.reshape(rows, -1)[sub].reshape(-1)
        for m in (3, 4):
            x = synth.random_activations(m, cols, seed=m + fmt + cols)
            got = dev.qmatmul(q, x)
            assert rel_err(got[:, sub], o.qmatmul(fmt, wsub, len(sub), cols, x)) <= 2e-5, (cols, m)
            try:
                dev.set_option("mmq.i8_min_m", 99)  # the vector kernels
                vector = dev.qmatmul(q, x)
            finally:
                dev.set_option("mmq.i8_min_m", 0)
            assert rel_err(got, vector) <= 2e-6, (cols, m)
            assert np.array_equal(got, vector) != tiles, (cols, m)


def test_config_q4_0_4096x4096(dev):
    # the single-QMatMul configuration: Q4_0 4096x4096, one f32 N(0,1) vector, seeded
    rows = cols = 4096
    w = synth.random_weight(synth.Q4_0, rows, cols, seed=20240)
    x = synth.random_activations(1, cols, seed=20241)
    q = dev.qtensor(synth.Q4_0, rows, cols, w)
    got = dev.qmatmul(q, x)
    sub = np.arange(0, rows, 16)  # the oracle on a row subset keeps the test in seconds
    wb = w.reshape(rows, -1)[sub].reshape(-1)
    want = o.qmatmul(synth.Q4_0, wb, len(sub), cols, x)
    assert rel_err(got[:, sub], want) <= 2e-5
    # and against candy's literal CPU composition (dequantize + naive f32 loops) on the
    # Q8_0-dequantized activations: same mathematics, different rounding
    xdq = o.dequantize(synth.Q8_0, o.quantize_q8_0(x)).reshape(1, cols)
    lit = o.matmul_dequant_f32(synth.Q4_0, wb, len(sub), cols, xdq)
    assert rel_err(got[:, sub], lit) <= 1e-4


@pytest.mark.parametrize("rows,cols,variant", [(64, 1024, 0), (48, 2048, 0),          # up to 8 super-blocks a row
                                               (4096, 4096, 1), (4096, 4096, 2),      # 16: one / two strips a wavefront
                                               (160, 6144, 0),                        # 24: three super-blocks a slice
                                               (96, 8192, 1), (96, 8192, 2),          # 32
                                               (128, 11008, 0),                       # 43: slices past the end of K
                                               (64, 12288, 0)])                       # 48: the longest row it takes
@pytest.mark.parametrize("m", [2, 3, 7, 16, 17, 25, 32])
def test_small_batch_int8_one_pass(dev, rows, cols, variant, m):
    # 2 .. 16 activation rows (up to 32, as two tiles of 16, for rows of up to 4096 values) against Q4_K on the
    # int8 matrix cores, one pass over the weights (the role of
    # mul_mat_vec_q<ncols_y>, quantized.cu:2787-2871): integer sub-block dots, scales applied as
    # vec_dot_q4_K_q8_1 does (quantized.cu:2239-2263); only the f32 summation order differs from the CPU loop
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=rows + cols + m)
    x = synth.random_activations(m, cols, seed=cols + 5 * m)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    try:
        dev.set_option("mmv.min_m", 2)
        dev.set_option("mmv.variant", variant)
        got = dev.qmatmul(q, x)
        dev.set_option("mmv.max_m", 0)
        other = dev.qmatmul(q, x)  # the vector / tile kernels on the same quantized activations
    finally:
        dev.set_option("mmv.min_m", 3), dev.set_option("mmv.max_m", 32), dev.set_option("mmv.variant", 0)
    assert got.shape == (m, rows)
    if rows * cols <= 1 << 21:
        want = o.qmatmul(synth.Q4_K, w, rows, cols, x)
    else:
        sub = np.arange(0, rows, rows // 128)
        want = o.qmatmul(synth.Q4_K, w.reshape(rows, -1)[sub].reshape(-1), len(sub), cols, x)
        got, other = got[:, sub], other[:, sub]
    assert rel_err(got, want) <= 2e-5
    assert rel_err(got, other) <= 2e-5
    q.free()


def test_small_batch_int8_one_pass_random_shapes(dev):
    # seeded random shapes over everything the kernel takes: 16 .. 640 weight rows in steps of 16, 1 .. 48
    # super-blocks per row, 2 .. 32 activation rows (more than 16 only up to 16 super-blocks), both strip variants
    rng = np.random.default_rng(2024)
    dev.set_option("mmv.min_m", 2)
    try:
        for case in range(48):
            nsb = int(rng.integers(1, 49))
            rows = 16 * int(rng.integers(1, 41))
            m = int(rng.integers(2, 33 if nsb <= 16 else 17))
            cols = 256 * nsb
            w = synth.random_weight(synth.Q4_K, rows, cols, seed=1000 + case)
            x = synth.random_activations(m, cols, seed=2000 + case)
            q = dev.qtensor(synth.Q4_K, rows, cols, w)
            dev.set_option("mmv.variant", int(rng.integers(0, 3)))
            got = dev.qmatmul(q, x)
            want = o.qmatmul(synth.Q4_K, w, rows, cols, x)
            assert got.shape == (m, rows) and rel_err(got, want) <= 2e-5, (case, rows, cols, m)
            xb = o.quantize_q8_0(x)     # and from Q8_0 blocks: the same quants, the same kernel, the same bits
            assert np.array_equal(dev.qmatmul_q8(q, xb, m).view(np.uint32), got.view(np.uint32)), (case, rows, cols, m)
            q.free()
    finally:
        dev.set_option("mmv.min_m", 3), dev.set_option("mmv.variant", 0)


def test_small_batch_int8_one_pass_leaves_other_shapes_alone(dev):
    # rows off the 16-row strips, rows longer than 48 super-blocks and other formats keep their kernels: same bits
    # whether the option is on or off
    for fmt, rows, cols in ((synth.Q4_K, 100, 4096), (synth.Q4_K, 64, 14336), (synth.Q6_K, 64, 4096), (synth.Q8_0, 64, 4096)):
        w = synth.random_weight(fmt, rows, cols, seed=rows + fmt)
        x = synth.random_activations(5, cols, seed=9)
        q = dev.qtensor(fmt, rows, cols, w)
        a = dev.qmatmul(q, x)
        dev.set_option("mmv.max_m", 0)
        try:
            b = dev.qmatmul(q, x)
        finally:
            dev.set_option("mmv.max_m", 32)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (fmt, rows, cols)
        assert rel_err(a, o.qmatmul(fmt, w, rows, cols, x)) <= 2e-5


@pytest.mark.parametrize("fmt", [synth.Q8_0, synth.Q4_K])
@pytest.mark.parametrize("rows,cols", [(4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)])
def test_config_sweep_full_shapes(dev, fmt, rows, cols):
    # the batch-1 sweep shapes at full size: oracle on a strided row subset + linearity over the whole output
    w = synth.random_weight(fmt, rows, cols, seed=rows + cols + fmt)
    x = synth.random_activations(1, cols, seed=3 * rows + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    sub = np.arange(0, rows, max(1, rows // 128))
    rb = synth.weight_nbytes(fmt, 1, cols)
    wb = w.reshape(rows, rb)[sub].reshape(-1)
    want = o.qmatmul(fmt, wb, len(sub), cols, x)
    assert rel_err(got[:, sub], want) <= 2e-5
    # exact scaling property over every row: x -> 2x doubles Q8_0 scales, leaves quants unchanged
    got2 = dev.qmatmul(q, 2 * x)
    assert np.array_equal(got2, 2 * got)


def test_q6_k_head_shape(dev):
    rows, cols = 32000, 4096
    w = synth.random_weight(synth.Q6_K, rows, cols, seed=606)
    x = synth.random_activations(1, cols, seed=607)
    q = dev.qtensor(synth.Q6_K, rows, cols, w)
    got = dev.qmatmul(q, x)
    sub = np.arange(0, rows, 250)
    wb = w.reshape(rows, -1)[sub].reshape(-1)
    assert rel_err(got[:, sub], o.qmatmul(synth.Q6_K, wb, len(sub), cols, x)) <= 2e-5


def test_q6_k_llama3_head_shape(dev):
    # the Llama-3 output head, 128256 x 4096 in Q6_K (431 MB), batch 1: oracle on a strided row subset, the exact
    # scaling property over every row
    rows, cols = 128256, 4096
    w = synth.random_weight(synth.Q6_K, rows, cols, seed=808)
    x = synth.random_activations(1, cols, seed=809)
    q = dev.qtensor(synth.Q6_K, rows, cols, w)
    got = dev.qmatmul(q, x)
    sub = np.arange(0, rows, 501)
    wb = w.reshape(rows, -1)[sub].reshape(-1)
    assert rel_err(got[:, sub], o.qmatmul(synth.Q6_K, wb, len(sub), cols, x)) <= 2e-5
    assert np.array_equal(dev.qmatmul(q, 2 * x), 2 * got)
    q.free()


def test_rows_past_the_small_batch_limit_are_an_error_not_a_fault(dev):
    # with fewer than 16 activation rows the quantized image of a row must fit LDS (about 49 900 values) unless the
    # batch-1 kernel takes it (Q4_K: up to 8 x 64 units = 32768 values... its image has the same limit): longer rows
    # are refused with a message, from 16 rows on the tile kernels have no such limit
    rows, cols = 16, 65536
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=3)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    for m in (1, 3, 15):
        x = synth.random_activations(m, cols, seed=m)
        try:
            got = dev.qmatmul(q, x)
        except hip.CandyHipError as e:
            assert "too large for the matvec kernel" in str(e), str(e)
        else:
            assert rel_err(got, o.qmatmul(synth.Q4_K, w, rows, cols, x)) <= 2e-5
    x = synth.random_activations(16, cols, seed=16)
    assert rel_err(dev.qmatmul(q, x), o.qmatmul(synth.Q4_K, w, rows, cols, x)) <= 2e-5
    dev.synchronize()  # the handle is still good
    q.free()


def test_qmatmul_from_prequantized_blocks(dev):
    rows, cols, m = 64, 1024, 3
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=1)
    x = synth.random_activations(m, cols, seed=2)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    xb = o.quantize_q8_0(x)
    assert np.array_equal(dev.qmatmul_q8(q, xb, m), dev.qmatmul(q, x))


def test_zero_and_extreme_activations(dev):
    rows, cols = 32, 512
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=4)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    assert np.all(dev.qmatmul(q, np.zeros((1, cols), np.float32)) == 0)
    x = synth.random_activations(1, cols, seed=5) * np.float32(1e4)
    assert rel_err(dev.qmatmul(q, x), o.qmatmul(synth.Q4_K, w, rows, cols, x)) <= 2e-5


def test_qmatmul_errors(dev):
    with pytest.raises(hip.CandyHipError, match="multiple of the block size"):
        dev.qtensor(synth.Q4_K, 4, 100, np.zeros(10, np.uint8))
    with pytest.raises(hip.CandyHipError, match="bytes"):
        dev.qtensor(synth.Q4_K, 4, 256, np.zeros(10, np.uint8))
    with pytest.raises(hip.CandyHipError, match="unknown quantized format"):
        dev.qtensor(99, 4, 256, np.zeros(10, np.uint8))
    with pytest.raises(hip.CandyHipError, match="invalid matrix dimensions"):
        dev.qtensor(synth.Q4_K, 0, 256, np.zeros(0, np.uint8))
