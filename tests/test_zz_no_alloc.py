"""The allocation-free contraction (candy_hip_qmatmul_noalloc) against candy_hip_qmatmul, through the C ABI.

Its quantized activations live in a file-scope device array that every call on the GPU shares, so the second
call of each pair is smaller than the first: whatever the first one left behind must not show."""
import ctypes

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
    shapes = [(big, 8), (small, 3), (big, 1), (small, 1), (big, 15), (small, 4)]
    if fmt == synth.Q4_K:  # one row against 4096 x 4096: candy_hip_qmatmul quantizes inside the contraction's launch there
        shapes.append((dev.qtensor(fmt, 4096, 4096, synth.random_weight(fmt, 4096, 4096, seed=902)), 1))
    for (w, m) in shapes:
        x = synth.random_activations(m, w.cols, seed=17 * m + w.cols)
        ref, got = both(dev, w, x)
        assert np.abs(ref).max() > 0
        if m <= 4:
            # the same vector kernels answer both calls: same bits
            assert np.array_equal(ref.view(np.uint32), got.view(np.uint32)), (fmt, m)
        else:
            # candy_hip_qmatmul may take the int8 tile kernel here: the same integer dots in another f32 summation order
            err = float(np.max(np.abs(got.astype(np.float64) - ref)) / np.max(np.abs(ref)))
            assert err <= 2e-6, (fmt, m, err)  # the bar is 1e-3; two evaluations of the same exact dots stay far inside it


@pytest.mark.parametrize("fmt", [synth.Q4_K, synth.Q8_0, synth.Q6_K, synth.Q4_0])
def test_against_the_cpu_oracle_on_a_handle_that_never_allocated(fmt):
    # A fresh device handle whose FIRST contraction is the allocation-free one: the handle's grow-only workspaces
    # (the only device memory candy_hip_qmatmul allocates on the way) must still be empty afterwards, and the
    # result is held to the CPU oracle, not to another device path: 1e-3 asked, 2e-5 expected of exact integer dots.
    d = hip.Device(0)
    try:
        L = hip.lib()
        for rows, cols, m in ((4096, 4096, 1), (512, 4096, 8), (200, 1024, 3)):
            blocks = synth.random_weight(fmt, rows, cols, seed=950 + fmt + m)
            w = d.qtensor(fmt, rows, cols, blocks)
            x = synth.random_activations(m, cols, seed=951 + m)
            src, dst = d.from_numpy(x), d.alloc(m * rows * 4)
            hip._check(L.candy_hip_qmatmul_noalloc(d.handle, w.handle, src.ptr, m, dst.ptr))
            got = dst.download(np.float32, m * rows).reshape(m, rows)
            assert d.get_option("runtime.workspace_bytes") == 0 and d.get_option("runtime.split_workspace_bytes") == 0
            want = o.qmatmul(fmt, blocks, rows, cols, x)
            err = float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))
            assert err <= 1e-3 and err <= 2e-5, (fmt, rows, cols, m, err)
        # the allocating entry point on the same handle does grow the workspace (the key reports it), same result
        hip._check(L.candy_hip_qmatmul(d.handle, w.handle, src.ptr, m, dst.ptr))
        assert d.get_option("runtime.workspace_bytes") > 0
        again = dst.download(np.float32, m * rows).reshape(m, rows)
        assert np.array_equal(got.view(np.uint32), again.view(np.uint32))
    finally:
        d.close()


def test_sizes_beyond_the_scratch_are_refused(dev):
    w = dev.qtensor(synth.Q8_0, 4, 65536, synth.random_weight(synth.Q8_0, 4, 65536, seed=5))
    x = dev.from_numpy(synth.random_activations(15, 65536, seed=6))
    y = dev.alloc(15 * 4 * 4)
    L = hip.lib()
    assert L.candy_hip_qmatmul_noalloc(dev.handle, w.handle, x.ptr, 16, y.ptr) == 1
    assert b"1 .. 15" in L.candy_hip_last_error()
    assert L.candy_hip_qmatmul_noalloc(dev.handle, w.handle, x.ptr, 15, y.ptr) == 1  # 15 x 65536 x 1.25 bytes > 1 MiB
    assert b"scratch" in L.candy_hip_last_error()
