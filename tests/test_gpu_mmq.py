"""GPU parity of the batched (m >= 16) QMatMul, the MFMA tile kernels, against the CPU oracle.
Bar: max|gpu - ref| / max|ref| <= 1e-3. The fp16 tile kernels (Q4_K / Q5_K / Q6_K / Q8_0 / Q4_0 from 256
activation rows up, the 32-value formats on wide prompt-sized grids) round their operands to fp16 and land near 3e-4;
the Q4_K / Q6_K / Q8_0 / Q4_0 int8 kernel multiplies integers on the matrix cores and differs from the oracle's
integer dots only by f32 summation order, so it is held to 2e-5."""
import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import oracle as o

pytestmark = pytest.mark.gpu
TOL = 1e-3


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def rel_err(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want.astype(np.float64))) / np.max(np.abs(want)))


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML])
@pytest.mark.parametrize("m", [16, 17, 33, 64, 100, 128, 200])
def test_tile_kernel_matches_oracle(dev, fmt, m):
    rows, cols = 200, 1024  # rows not a multiple of any tile width, cols = 4 super-blocks
    w = synth.random_weight(fmt, rows, cols, seed=m + fmt)
    x = synth.random_activations(m, cols, seed=m * 5 + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (m, rows)
    assert rel_err(got, want) <= TOL
    # every row on its own is within the bar too (no row may hide behind a large neighbour)
    per_row = np.max(np.abs(got - want), axis=1) / np.max(np.abs(want), axis=1)
    assert np.max(per_row) <= 2 * TOL


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML, synth.Q4_1,
                                 synth.Q4_1_GGML, synth.Q5_0, synth.Q5_1, synth.Q5_K, synth.Q2_K, synth.Q3_K])
@pytest.mark.parametrize("m", [16, 31, 32, 48, 65, 129, 300])
@pytest.mark.parametrize("rows,cols", [(1, 256), (15, 768), (67, 1280), (130, 2304), (1030, 512)])
def test_int8_tiles_are_integer_exact(dev, fmt, m, rows, cols):
    # rows off every 4/16/64 boundary, block counts off every stage length, m off every tile height
    w = synth.random_weight(fmt, rows, cols, seed=rows + m)
    x = synth.random_activations(m, cols, seed=cols + m)
    # single Q4_K contractions move to the fp16 tiles from 33 rows on; here the int8 tiles are asked for up to the
    # decoder's threshold (what its prompt pass uses)
    dev.set_option("mmq.f16_api_min_m", 256)
    try:
        got = dev.qmatmul(dev.qtensor(fmt, rows, cols, w), x)
    finally:
        dev.set_option("mmq.f16_api_min_m", 33)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (m, rows)
    # 256 activation rows or more run on the fp16 tiles (operands rounded to fp16)
    assert rel_err(got, want) <= (5e-4 if m >= 256 and fmt in (synth.Q4_K, synth.Q6_K, synth.Q5_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML) else 2e-5)


@pytest.mark.parametrize("m", [33, 48, 64, 65, 96, 100, 128, 129, 200, 255])
@pytest.mark.parametrize("rows,cols", [(1, 256), (127, 512), (129, 1024), (300, 2304), (1030, 768), (130, 4352)])
def test_q4k_fp16_tiles_from_33_rows(dev, m, rows, cols):
    # a single Q4_K contraction of 33 .. 255 rows: 128 x 128 tiles up to 128 rows, 128 x 256 above, K split over
    # workgroups on small grids; fp16 operands (the bar of the big tiles), the same bits from call to call
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=7 * rows + m)
    x = synth.random_activations(m, cols, seed=cols + 3 * m)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    got = dev.qmatmul(q, x)
    err = rel_err(got, o.qmatmul(synth.Q4_K, w, rows, cols, x))
    assert err <= 5e-4, err
    assert np.array_equal(got, dev.qmatmul(q, x))


@pytest.mark.parametrize("fmt", [synth.Q6_K, synth.Q5_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML])
@pytest.mark.parametrize("m", [33, 64, 65, 128, 129, 255])
@pytest.mark.parametrize("rows,cols", [(127, 512), (300, 2304), (1030, 768)])
def test_other_formats_fp16_tiles_from_65_rows(dev, fmt, m, rows, cols):
    # a single contraction of the other formats: up to 64 rows one tile of the integer-exact kernel, from 65 rows the
    # fp16 tiles (128 x 128 up to 128 rows), at their bar and not at the exact kernel's
    w = synth.random_weight(fmt, rows, cols, seed=5 * rows + m + fmt)
    x = synth.random_activations(m, cols, seed=cols + m)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    err = rel_err(got, o.qmatmul(fmt, w, rows, cols, x))
    if m <= 64 and fmt != synth.Q6_K:  # Q6_K is on the fp16 tiles from 33 rows, like Q4_K
        assert err <= 2e-5, err
    else:
        assert 2e-6 < err <= 5e-4, err
    assert np.array_equal(got, dev.qmatmul(q, x))


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q5_K, synth.Q8_0, synth.Q4_0])
def test_single_contractions_stay_exact_on_request(dev, fmt):
    # "mmq.f16_api_min_m" = 1 << 30 keeps candy_hip_qmatmul on the integer-exact kernels at every batch size
    rows, cols, m = 300, 1024, 400
    w = synth.random_weight(fmt, rows, cols, seed=fmt + 1)
    x = synth.random_activations(m, cols, seed=fmt + 2)
    q = dev.qtensor(fmt, rows, cols, w)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert rel_err(dev.qmatmul(q, x), want) > 2e-6  # by default: fp16 tiles
    dev.set_option("mmq.f16_api_min_m", 1 << 30)
    try:
        assert rel_err(dev.qmatmul(q, x), want) <= 2e-6
    finally:
        dev.set_option("mmq.f16_api_min_m", 33)


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K])
@pytest.mark.parametrize("rows,cols", [(200, 11008), (64, 4352), (1000, 2560)])
def test_int8_tiles_split_the_contraction_on_small_grids(dev, monkeypatch, fmt, rows, cols):
    # few weight rows and a long contraction: the grid is at most one wavefront per SIMD, so K is split over
    # workgroups and the copies are summed in a
    # fixed order: the answer moves by f32 summation order only, and is the same from call to call
    w = synth.random_weight(fmt, rows, cols, seed=rows + cols + fmt)
    q = dev.qtensor(fmt, rows, cols, w)
    dev.set_option("mmv.max_m", 0)  # 16 .. 32 rows of Q4_K on the tile kernel here, not on the one-pass kernel
    dev.set_option("mmq.f16_api_min_m", 256)  # ... and 33 rows and more not on the fp16 tiles
    try:
        for m in (16, 24, 33, 64, 130):
            x = synth.random_activations(m, cols, seed=m * 7 + fmt)
            got = dev.qmatmul(q, x)
            assert np.array_equal(got.view(np.uint32), dev.qmatmul(q, x).view(np.uint32))
            if m in (16, 33):
                assert rel_err(got, o.qmatmul(fmt, w, rows, cols, x)) <= 2e-5, m
            dev.set_option("mmq.i8_grid_split", 0)
            try:
                whole = dev.qmatmul(q, x)
            finally:
                dev.set_option("mmq.i8_grid_split", 1)
            assert rel_err(got, whole) <= 2e-6, m
    finally:
        dev.set_option("mmv.max_m", 32)
        dev.set_option("mmq.f16_api_min_m", 33)


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q5_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML])
@pytest.mark.parametrize("m", [256, 257, 300, 512, 700])
@pytest.mark.parametrize("rows,cols", [(1, 256), (127, 512), (129, 1024), (300, 2304), (1030, 768), (130, 4352)])
def test_big_fp16_tiles(dev, fmt, m, rows, cols):
    # rows off the 128-row tile, m off the 256-row tile, odd and even super-block counts; the few-tile
    # shapes split K over several workgroups (17 super-blocks: uneven splits)
    w = synth.random_weight(fmt, rows, cols, seed=3 * rows + m)
    x = synth.random_activations(m, cols, seed=cols + 7 * m)
    got = dev.qmatmul(dev.qtensor(fmt, rows, cols, w), x)
    want = o.qmatmul(fmt, w, rows, cols, x)
    assert got.shape == (m, rows)
    assert rel_err(got, want) <= 5e-4  # observed 3e-4; a dropped block or a wrong scale costs far more
    if rows >= 100:  # per activation row (a max over few outputs is no scale to measure against)
        per_row = np.max(np.abs(got - want), axis=1) / np.max(np.abs(want), axis=1)
        assert np.max(per_row) <= 2 * TOL


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q6_K, synth.Q5_K, synth.Q8_0, synth.Q4_0, synth.Q4_0_GGML])
@pytest.mark.parametrize("m,rows,cols", [(256, 128, 256), (300, 129, 1024), (513, 1030, 768), (700, 130, 4352),
                                         (260, 2100, 512), (96, 300, 2304), (128, 1030, 768), (200, 25000, 256)])
def test_role_split_tiles_equal_the_single_role_tiles(dev, fmt, m, rows, cols):
    # 128 x 256 tiles (and Q4_K's 128 x 128 ones: up to 128 rows, and 129-256 rows on many weight rows): producer /
    # consumer wavefronts (the default) and the kernel whose wavefronts do both run the same multiply-adds in the
    # same order on the same fp16 operands, with and without a K split.  Below the fp16 threshold of a format both
    # runs take the same int8 tiles.
    w = synth.random_weight(fmt, rows, cols, seed=rows + 3 * m)
    x = synth.random_activations(m, cols, seed=cols + m)
    q = dev.qtensor(fmt, rows, cols, w)
    got = dev.qmatmul(q, x)
    dev.set_option("mmq.f16_shape", 3)
    try:
        single = dev.qmatmul(q, x)
    finally:
        dev.set_option("mmq.f16_shape", 0)
    assert np.array_equal(got.view(np.uint32), single.view(np.uint32))


@pytest.mark.parametrize("m,rows,cols", [(512, 1792, 1024), (128, 3584, 768), (300, 112, 512), (257, 2240, 2304),
                                         (1000, 14336, 256)])
@pytest.mark.parametrize("split", [1, 2])
def test_tiles_of_112_weight_rows_equal_tiles_of_128(dev, m, rows, cols, split):
    # Q4_K row counts that 112 divides (14336 = 128 * 112) take tiles of 112 weight rows where those fill the chip
    # better: the same multiply-adds in the same order as the 128-row tiles when K is split the same way, and the
    # oracle's values on every row (default split)
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=rows + m)
    x = synth.random_activations(m, cols, seed=cols + 2 * m)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    dev.set_option("mmq.f16_split", split)
    try:
        got = dev.qmatmul(q, x)
        dev.set_option("mmq.f16_shape", 4)
        wide = dev.qmatmul(q, x)
    finally:
        dev.set_option("mmq.f16_shape", 0)
        dev.set_option("mmq.f16_split", 0)
    assert np.array_equal(got.view(np.uint32), wide.view(np.uint32))
    if split == 1 and rows * m <= 1 << 20:
        assert rel_err(dev.qmatmul(q, x), o.qmatmul(synth.Q4_K, w, rows, cols, x)) <= 5e-4


def test_q8_0_wide_prompt_grid_takes_the_fp16_tiles(dev):
    # many weight rows and a prompt-sized batch: Q8_0 leaves the int8 tiles for the 128 x 128 fp16 tiles
    rows, cols, m = 8192, 256, 352
    w = synth.random_weight(synth.Q8_0, rows, cols, seed=9)
    x = synth.random_activations(m, cols, seed=10)
    got = dev.qmatmul(dev.qtensor(synth.Q8_0, rows, cols, w), x)
    err = rel_err(got, o.qmatmul(synth.Q8_0, w, rows, cols, x))
    assert 2e-6 < err <= TOL  # fp16 operands: not the integer-exact kernel


@pytest.mark.parametrize("fmt,rows,cols", [(synth.Q8_0, 70, 96), (synth.Q4_0, 33, 160), (synth.Q8_0, 64, 32)])
def test_contraction_length_not_a_multiple_of_64(dev, fmt, rows, cols):
    # odd block counts take the small-batch kernel in slices: same result, integer-exact dots
    m = 20
    w = synth.random_weight(fmt, rows, cols, seed=rows)
    x = synth.random_activations(m, cols, seed=cols)
    got = dev.qmatmul(dev.qtensor(fmt, rows, cols, w), x)
    assert rel_err(got, o.qmatmul(fmt, w, rows, cols, x)) <= 2e-5


@pytest.mark.parametrize("m", [16, 128, 512])
def test_config_prefill_q4k_14336x4096(dev, m):
    # the batched-prefill configuration (Q4_K 14336x4096, M in {16, 128, 512}) at full size; the oracle runs on a strided subset of the weight rows
    rows, cols = 14336, 4096
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=77)
    x = synth.random_activations(m, cols, seed=78 + m)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    got = dev.qmatmul(q, x)
    sub = np.arange(0, rows, 223)  # 65 rows, at varying places of the 16-, 112- and 128-row units the kernels tile by
    rb = synth.weight_nbytes(synth.Q4_K, 1, cols)
    want = o.qmatmul(synth.Q4_K, w.reshape(rows, rb)[sub].reshape(-1), len(sub), cols, x)
    assert rel_err(got[:, sub], want) <= TOL
    # size-independent properties over the whole output:
    # (1) x -> 2x doubles every Q8_0 scale and leaves the quants alone, so the result doubles exactly
    assert np.array_equal(dev.qmatmul(q, 2 * x), 2 * got)
    # (2) the batch-1 kernel (integer dots) on single rows agrees with the tile kernel's rows
    for r in (0, m - 1):
        assert rel_err(got[r:r + 1], dev.qmatmul(q, x[r:r + 1])) <= TOL


@pytest.mark.parametrize("m", [64, 512])
def test_mixed_format_prefill_q6k_down_proj(dev, m):
    rows, cols = 4096, 14336
    w = synth.random_weight(synth.Q6_K, rows, cols, seed=5)
    x = synth.random_activations(m, cols, seed=6)
    q = dev.qtensor(synth.Q6_K, rows, cols, w)
    got = dev.qmatmul(q, x)
    sub = np.arange(0, rows, 128)
    rb = synth.weight_nbytes(synth.Q6_K, 1, cols)
    want = o.qmatmul(synth.Q6_K, w.reshape(rows, rb)[sub].reshape(-1), len(sub), cols, x)
    assert rel_err(got[:, sub], want) <= TOL
    # split-K partial sums are added in a fixed order: the same call gives the same bits
    assert np.array_equal(got, dev.qmatmul(q, x))


def test_batch_size_boundaries_agree_within_their_bars(dev):
    # Which kernel contracts depends on the number of activation rows.  Rows computed in a batch of one size and
    # again in a batch across the next boundary agree to f32 summation order where both kernels are integer-exact
    # (2 | 3: vector | one-pass; 16 | 17: one tile | two tiles) and to the fp16-operand bar across the fp16
    # threshold (32 | 33 for a single Q4_K contraction).
    rows, cols = 512, 2048
    w = synth.random_weight(synth.Q4_K, rows, cols, seed=41)
    q = dev.qtensor(synth.Q4_K, rows, cols, w)
    x = synth.random_activations(33, cols, seed=42)
    want = o.qmatmul(synth.Q4_K, w, rows, cols, x)
    for lo, hi, bar in ((2, 3, 2e-6), (16, 17, 2e-6), (32, 33, 1e-3)):
        a, b = dev.qmatmul(q, x[:lo]), dev.qmatmul(q, x[:hi])
        d = rel_err(b[:lo], a.astype(np.float64))
        assert d <= bar, (lo, hi, d)
        assert rel_err(a, want[:lo]) <= 2e-5                      # below the threshold: exact kernels
        assert rel_err(b, want[:hi]) <= (5e-4 if hi >= 33 else 2e-5)
    a, b = dev.qmatmul(q, x[:32]), dev.qmatmul(q, x[:33])
    assert rel_err(b[:32], a.astype(np.float64)) > 1e-6           # and it IS another kernel: not the same bits
