"""The allocation-free contraction (candy_hip_qmatmul_noalloc) against candy_hip_qmatmul, through the C ABI.

Its quantized activations live in a file-scope device array that every call on the GPU shares, so the second
call of each pair is smaller than the first: whatever the first one left behind must not show."""
import ctypes

import numpy as np
import pytest

from candy_amd import hip, synth

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def both(dev, w, x):
    """(candy_hip_qmatmul, candy_hip_qmatmul_noalloc) on the same device buffers."""
    m = x.shape[0]
    src = dev.from_numpy(x)
    outs = []
    for fn in (hip.lib().candy_hip_qmatmul, hip.lib().candy_hip_qmatmul_noalloc):
        dst = dev.alloc(m * w.rows * 4)
        hip._check(hip.lib().candy_hip_zero(dev.handle, dst.ptr, dst.nbytes))
        hip._check(fn(dev.handle, w.handle, src.ptr, m, dst.ptr))
        outs.append(dst.download(np.float32, m * w.rows).reshape(m, w.rows))
    return outs


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q8_0, synth.Q6_K, synth.Q4_0])
def test_two_calls_in_a_row_second_smaller(dev, fmt):
    big = dev.qtensor(fmt, 512, 4096, synth.random_weight(fmt, 512, 4096, seed=900 + fmt))
    small = dev.qtensor(fmt, 200, 1024, synth.random_weight(fmt, 200, 1024, seed=901 + fmt))
    for (w, m) in ((big, 8), (small, 3), (big, 1), (small, 1), (big, 15), (small, 4)):
        x = synth.random_activations(m, w.cols, seed=17 * m + w.cols)
        ref, got = both(dev, w, x)
        assert np.abs(ref).max() > 0
        if m <= 4:
            # the same vector kernels answer both calls: same bits
            assert np.array_equal(ref.view(np.uint32), got.view(np.uint32)), (fmt, m)
        else:
            # candy_hip_qmatmul may take the int8 tile kernel here: the same integer dots in another f32 summation order
            err = float(np.max(np.abs(got.astype(np.float64) - ref)) / np.max(np.abs(ref)))
            assert err <= 1e-3, (fmt, m, err)
            assert err <= 2e-6, (fmt, m, err)


def test_sizes_beyond_the_scratch_are_refused(dev):
    w = dev.qtensor(synth.Q8_0, 4, 65536, synth.random_weight(synth.Q8_0, 4, 65536, seed=5))
    x = dev.from_numpy(synth.random_activations(15, 65536, seed=6))
    y = dev.alloc(15 * 4 * 4)
    L = hip.lib()
    assert L.candy_hip_qmatmul_noalloc(dev.handle, w.handle, x.ptr, 16, y.ptr) == 1
    assert b"1 .. 15" in L.candy_hip_last_error()
    assert L.candy_hip_qmatmul_noalloc(dev.handle, w.handle, x.ptr, 15, y.ptr) == 1  # 15 x 65536 x 1.25 bytes > 1 MiB
    assert b"scratch" in L.candy_hip_last_error()
