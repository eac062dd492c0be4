"""GPU parity of the f32 decode-step ops against the CPU oracle and the reference's own
test vectors. Tolerances: the reference's tests use abs diff < 1e-6 on O(1) values; parallel
reductions and f32 exp/sqrt on the device stay inside a relative 1e-5."""
import math

import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import oracle as o

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def close(a, b, rtol=1e-5, atol=1e-6):
    a, b = np.asarray(a, np.float64).reshape(-1), np.asarray(b, np.float64).reshape(-1)
    return a.shape == b.shape and (a.size == 0 or np.all(np.abs(a - b) <= atol + rtol * np.abs(b)))


def test_reference_vectors(dev, golden):
    for c in golden["fast_rms_norm_f32"]:
        assert close(dev.rms_norm(c["src"], c["dims"][-1], c["eps"], c["alpha"]), c["want"], 0, 1e-6), c["name"]
    for c in golden["rope_f32"]:
        assert close(dev.rope(c["src"], c["cos"], c["sin"], c["bh"], c["td"], c["d"], c["stride_b"]), c["want"], 0, 1e-6), c["name"]
    for c in golden["rope_i_f32"]:
        assert close(dev.rope_i(c["src"], c["cos"], c["sin"], c["bh"], c["td"], c["stride_b"]), c["want"], 0, 1e-6), c["name"]
    for c in golden["rope_thd_f32"]:
        assert close(dev.rope_thd(c["src"], c["cos"], c["sin"], c["b"], c["t"], c["h"], c["d"], c["stride_b"]), c["want"], 0, 1e-6), c["name"]
    for c in golden["fast_softmax_f32"]:
        assert close(dev.softmax(c["src"], c["dims"][-1]), c["want"], 0, 1e-6), c["name"]
    for c in golden["fast_argmax_f32"]:
        if c["src"]:
            assert list(dev.argmax(c["src"], c["dims"][-1])) == c["want"], c["name"]
    for c in golden["matmul_f32"]:
        if c["m"]:
            assert close(dev.matmul_f32(c["a"], c["b"], 1, c["m"], c["n"], c["k"]), c["want"], 0, 1e-6), c["name"]
    for c in golden["silu_f32"]:
        want = [x / (1 + math.exp(-x)) for x in c["inp"]]
        assert close(dev.silu(c["inp"]), want, 0, 1e-6), c["name"]


def test_matmul_f32_strided_views_match_the_cpu_loop_bitwise(dev):
    # one batch through arbitrary (row, column) strides and start offsets: the call CpuStorage.MatMul makes for any
    # non-contiguous layout (cpu/storage.go:893-910 -> conv.go:373-389)
    rng = np.random.default_rng(11)
    m, n, k = 7, 33, 50
    abuf = rng.standard_normal(5 + m * k * 2).astype(np.float32)
    bbuf = rng.standard_normal(9 + k * n * 3).astype(np.float32)
    for (ast, bst, ao, bo) in (((k, 1), (1, k), 0, 0),           # Linear: contiguous x, W^T view
                               ((1, m), (n, 1), 5, 0),           # transposed lhs with an offset
                               ((2 * k, 2), (3, 3 * k), 3, 9),   # every-other-column lhs, strided W^T view, both offset
                               ((k, 1), (0, 1), 0, 2)):          # broadcast rows of rhs (stride 0)
        got = dev.matmul_f32_strided(abuf, bbuf, m, n, k, ast, bst, ao, bo)
        want = o.naive_batched_matmul_strided_f32(1, m, n, k, abuf[ao:], bbuf[bo:], [0, ast[0], ast[1]],
                                                  [0, bst[0], bst[1]], [0, n, 1], m * n)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (ast, bst)
    with pytest.raises(hip.CandyHipError, match="negative strides"):
        dev.matmul_f32_strided(abuf, bbuf, m, n, k, (k, -1), (n, 1))


def test_index_select_out_of_range_ids_are_reported_not_read(dev):
    # indexing.go:8-26 panics on an id outside the table (Go bounds check); the kernels read nothing there, write
    # zeros, and the next synchronising call on the handle fails
    table = np.arange(12, dtype=np.float32).reshape(4, 3)
    ids = np.array([2, 0x7FFFFFFFFFFFFFFF, 0], np.int64)
    assert np.array_equal(dev.index_select(table, ids), np.stack([table[2], np.zeros(3, np.float32), table[0]]))
    for bad in (4, -1, 1 << 40):
        dt, di = dev.from_numpy(table), dev.from_numpy(np.array([1, bad], np.int64))
        out = dev.alloc(2 * 3 * 4)
        hip._check(hip.lib().candy_hip_index_select(dev.handle, dt.ptr, 4, 3, di.ptr, 2, out.ptr))
        with pytest.raises(hip.CandyHipError, match="outside its table"):
            dev.synchronize()
        dev.synchronize()  # reported once, then clear
        got = out.download(np.float32, 6).reshape(2, 3)
        assert np.array_equal(got[0], table[1]) and not got[1].any()
    w = synth.random_weight(synth.Q8_0, 4, 64, seed=3)
    q = dev.qtensor(synth.Q8_0, 4, 64, w)
    di = dev.from_numpy(np.array([3, 4], np.int64))
    out = dev.alloc(2 * 64 * 4)
    hip._check(hip.lib().candy_hip_qindex_select(dev.handle, q.handle, di.ptr, 2, out.ptr))
    with pytest.raises(hip.CandyHipError, match="outside its table"):
        out.download(np.float32, 128)
    dev.synchronize()


def test_matmul_f32_matches_naive_loop_bitwise(dev):
    rng = np.random.default_rng(0)
    b, m, n, k = 2, 5, 300, 129
    a = rng.standard_normal((b, m, k)).astype(np.float32)
    bm = rng.standard_normal((b, k, n)).astype(np.float32)
    got = dev.matmul_f32(a, bm, b, m, n, k)
    want = o.naive_batched_matmul_f32(b, m, n, k, a, bm)
    # same accumulation order (l ascending, one f32 accumulator), products rounded before the add: the same bits
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    wt = rng.standard_normal((n, k)).astype(np.float32)  # Linear's transposed weight view
    got_t = dev.matmul_f32(a[0], wt, 1, m, n, k, rhs_transposed=True)
    want_t = o.naive_batched_matmul_strided_f32(1, m, n, k, a[0], wt, [0, k, 1], [0, 1, k], [0, n, 1], m * n)
    assert np.array_equal(got_t.view(np.uint32), want_t.view(np.uint32))
    with pytest.raises(hip.CandyHipError, match="invalid matrix dimensions"):
        dev.matmul_f32(a, bm, 1, 0, n, k)


@pytest.mark.parametrize("rows,cols", [(1, 4096), (7, 1000), (3, 11008)])
def test_rms_norm(dev, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = (rng.standard_normal((rows, cols)) * 3).astype(np.float32)
    alpha = rng.standard_normal(cols).astype(np.float32)
    assert close(dev.rms_norm(x, cols, 1e-5, alpha), o.fast_rms_norm(x, cols, 1e-5, alpha))
    assert close(dev.rms_norm(x, cols, 1e-5), o.fast_rms_norm(x, cols, 1e-5))


def test_rope_decode_and_prefill_shapes(dev):
    rng = np.random.default_rng(1)
    for bh, t, d in [(32, 1, 128), (8, 1, 128), (4, 9, 64)]:
        src = rng.standard_normal(bh * t * d).astype(np.float32)
        ang = rng.standard_normal((t, d // 2))
        cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        got = dev.rope(src, cos, sin, bh, t * d, d)
        assert np.array_equal(got, o.rope(src, cos, sin, bh, t * d, d)) or close(got, o.rope(src, cos, sin, bh, t * d, d))


def test_rope_i_and_rope_thd_match_oracle(dev):
    # RopeI (adjacent pairs) and RopeThd ([b, t, h, d] layout) against the CPU loops, with one table for all batch
    # entries and with one per entry; the device may fuse the multiply and the add, so a last-place difference is allowed
    rng = np.random.default_rng(3)
    for b, h, t, d in [(1, 32, 1, 128), (2, 8, 7, 64), (3, 4, 33, 128)]:
        src = rng.standard_normal(b * h * t * d).astype(np.float32)
        for per_batch in (False, True):
            ang = rng.standard_normal((b if per_batch else 1, t, d // 2))
            cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
            sb = h * t * d if per_batch else 0
            assert close(dev.rope_i(src, cos, sin, b * h, t * d, sb), o.rope_i(src, cos, sin, b * h, t * d, sb))
            assert close(dev.rope_thd(src, cos, sin, b, t, h, d, sb), o.rope_thd(src, cos, sin, b, t, h, d, sb))
    with pytest.raises(hip.CandyHipError, match="even"):
        dev.rope_thd(np.zeros(6, np.float32), np.zeros(3, np.float32), np.zeros(3, np.float32), 1, 2, 1, 3)


@pytest.mark.parametrize("rows,cols", [(32, 2049), (1, 32000), (5, 17)])
def test_softmax(dev, rows, cols):
    rng = np.random.default_rng(cols)
    x = (rng.standard_normal((rows, cols)) * 4).astype(np.float32)
    got = dev.softmax(x, cols)
    # the CPU loop adds `cols` exponentials into one f32 accumulator; over 32000 terms that
    # sequential sum drifts a few 1e-5 (relative) from the device's tree sum
    assert close(got, o.fast_softmax(x, cols), 1e-4, 1e-9)
    e = np.exp(x.astype(np.float64).reshape(rows, cols) - x.reshape(rows, cols).max(1, keepdims=True))
    assert close(got, e / e.sum(1, keepdims=True), 2e-6, 1e-12)  # and it is the accurate one
    assert close(got.reshape(rows, cols).sum(1), np.ones(rows), 1e-5)


def test_elementwise(dev):
    rng = np.random.default_rng(2)
    a = (rng.standard_normal(11008) * 5).astype(np.float32)
    b = rng.standard_normal(11008).astype(np.float32)
    assert np.array_equal(dev.add(a, b), o.add(a, b))
    assert np.array_equal(dev.mul(a, b), o.mul(a, b))
    assert close(dev.silu(a), o.silu(a), 1e-6, 1e-7)
    assert close(dev.silu_mul(a, b), o.mul(o.silu(a), b), 2e-6, 1e-7)


def test_argmax_first_maximum_wins(dev):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((4, 32000)).astype(np.float32)
    x[0, 5] = x[0, 31999] = 10.0          # tie: lowest index
    x[1, :] = -1.0                        # all equal
    x[2, 31999] = 50.0                    # last element
    assert list(dev.argmax(x, 32000)) == list(o.fast_argmax(x, 32000))
    assert list(dev.argmax(x, 32000))[:3] == [5, 0, 31999]


@pytest.mark.parametrize("cols", [128256, 32001, 4099, 7, 1])
def test_argmax_wide_and_ragged_rows(dev, cols):
    # rows wider than one pass of the block, widths that are not a multiple of 4 (rows then start
    # off a 16-byte boundary), ties on both sides of a vector boundary
    rng = np.random.default_rng(cols)
    x = rng.standard_normal((3, cols)).astype(np.float32)
    x[1, cols - 1] = 99.0
    x[1, cols // 2] = 99.0
    x[2, :] = np.float32(-np.inf)      # reduce.go:846-862: nothing beats -MaxFloat32 -> 0
    got = list(dev.argmax(x, cols))
    assert got == list(o.fast_argmax(x, cols))
    assert got[1] == cols // 2 and got[2] == 0


def test_index_select(dev):
    rng = np.random.default_rng(4)
    table = rng.standard_normal((50, 96)).astype(np.float32)
    ids = np.array([7, 0, 49, 7], np.int64)
    assert np.array_equal(dev.index_select(table, ids), table[ids])


@pytest.mark.parametrize("n_heads,n_kv,hd,n_pos,cap", [(32, 32, 128, 2049, 2304), (32, 8, 128, 640, 640),
                                                        (8, 2, 64, 37, 40), (4, 4, 128, 1, 8)])
def test_attention_decode(dev, n_heads, n_kv, hd, n_pos, cap):
    rng = np.random.default_rng(n_pos)
    q = rng.standard_normal((n_heads, hd)).astype(np.float32)
    k = rng.standard_normal((n_kv, cap, hd)).astype(np.float32)
    v = rng.standard_normal((n_kv, cap, hd)).astype(np.float32)
    scale = 1 / math.sqrt(hd)
    got = dev.attention_decode(q, k, v, n_heads, n_kv, hd, n_pos, cap * hd, scale)
    want = o.attention_decode(q, k, v, n_heads, n_kv, hd, n_pos, cap * hd, scale)
    assert close(got, want, 1e-4, 1e-5)
