"""Pins the oracle's f32 glue ops (matmul, RMSNorm, RoPE, softmax, SiLU, argmax, index-select,
attention) against the reference's own test vectors (tests/golden/candy_cpu_kernels.json)
and float64 closed forms."""
import math

import numpy as np

from oracle import oracle as o


def _close(a, b, tol):
    a, b = np.asarray(a, np.float64).reshape(-1), np.asarray(b, np.float64).reshape(-1)
    return a.shape == b.shape and (a.size == 0 or np.max(np.abs(a - b)) < tol)


def test_naive_matmul_reference_vectors(golden):
    for c in golden["matmul_f32"]:
        got = o.naive_batched_matmul_f32(1, c["m"], c["n"], c["k"], c["a"], c["b"])
        assert _close(got, c["want"], golden["tolerance"]), c["name"]
        m, n, k = c["m"], c["n"], c["k"]
        got_s = o.naive_batched_matmul_strided_f32(1, m, n, k, c["a"], c["b"], [0, k, 1], [0, n, 1], [0, n, 1], m * n)
        assert np.array_equal(got_s, got), c["name"]


def test_strided_matmul_reads_transposed_weight_view():
    # nn.Linear hands MatMul the weight [n, k] viewed as [k, n] with strides {1, k} (cpu/storage.go:892-909)
    rng = np.random.default_rng(0)
    m, n, k = 3, 5, 7
    a = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.standard_normal((n, k)).astype(np.float32)
    got = o.naive_batched_matmul_strided_f32(1, m, n, k, a, w, [0, k, 1], [0, 1, k], [0, n, 1], m * n)
    want = o.naive_batched_matmul_f32(1, m, n, k, a, np.ascontiguousarray(w.T))
    assert np.array_equal(got, want)
    assert _close(got, (a.astype(np.float64) @ w.T.astype(np.float64)), 1e-5)


def test_rms_norm_reference_vectors(golden):
    for c in golden["fast_rms_norm_f32"]:
        got = o.fast_rms_norm(c["src"], c["dims"][-1], c["eps"], c["alpha"])
        assert _close(got, c["want"], golden["tolerance"]), c["name"]


def test_rope_reference_vectors(golden):
    for c in golden["rope_f32"]:
        got = o.rope(c["src"], c["cos"], c["sin"], c["bh"], c["td"], c["d"], c["stride_b"])
        assert _close(got, c["want"], golden["tolerance"]), c["name"]


def test_rope_is_a_rotation_of_half_split_pairs():
    rng = np.random.default_rng(1)
    bh, t, d = 3, 5, 8
    src = rng.standard_normal((bh, t, d)).astype(np.float32)
    ang = rng.standard_normal((t, d // 2))
    got = o.rope(src, np.cos(ang), np.sin(ang), bh, t * d, d).reshape(bh, t, d).astype(np.float64)
    x1, x2 = src[..., : d // 2].astype(np.float64), src[..., d // 2:].astype(np.float64)
    assert _close(got[..., : d // 2], x1 * np.cos(ang) - x2 * np.sin(ang), 1e-5)
    assert _close(got[..., d // 2:], x1 * np.sin(ang) + x2 * np.cos(ang), 1e-5)
    assert _close(np.sum(got ** 2, -1), np.sum(src.astype(np.float64) ** 2, -1), 1e-4)  # norm preserved


def test_rope_i_and_rope_thd_reference_vectors(golden):
    for c in golden["rope_i_f32"]:
        got = o.rope_i(c["src"], c["cos"], c["sin"], c["bh"], c["td"], c["stride_b"])
        assert _close(got, c["want"], golden["tolerance"]), c["name"]
    for c in golden["rope_thd_f32"]:
        got = o.rope_thd(c["src"], c["cos"], c["sin"], c["b"], c["t"], c["h"], c["d"], c["stride_b"])
        assert _close(got, c["want"], golden["tolerance"]), c["name"]


def test_rope_i_rotates_adjacent_pairs_and_rope_thd_is_rope_on_the_transposed_layout():
    rng = np.random.default_rng(2)
    b, h, t, d = 2, 3, 5, 8
    ang = rng.standard_normal((t, d // 2))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    # rope_i: pair (2i, 2i + 1) of every row of t*d values turns by the angle of pair i (float64 closed form)
    src = rng.standard_normal((b * h, t, d // 2, 2)).astype(np.float32)
    got = o.rope_i(src, cos, sin, b * h, t * d).reshape(b * h, t, d // 2, 2).astype(np.float64)
    x, y = src[..., 0].astype(np.float64), src[..., 1].astype(np.float64)
    assert _close(got[..., 0], x * np.cos(ang) - y * np.sin(ang), 1e-5)
    assert _close(got[..., 1], x * np.sin(ang) + y * np.cos(ang), 1e-5)
    # per-batch tables (stride_b = elements per batch entry): batch entry i takes table i
    ang2 = rng.standard_normal((b, t, d // 2))
    cos2, sin2 = np.cos(ang2).astype(np.float32), np.sin(ang2).astype(np.float32)
    got2 = o.rope_i(src, cos2, sin2, b * h, t * d, stride_b=h * t * d).reshape(b, h, t, d // 2, 2)
    for i in range(b):
        want = o.rope_i(src.reshape(b, h, t, d // 2, 2)[i], cos2[i], sin2[i], h, t * d).reshape(h, t, d // 2, 2)
        assert np.array_equal(got2[i], want)
    # rope_thd on [b, t, h, d] is rope on [b, h, t, d] with the two middle axes swapped: same products, same bits
    src4 = rng.standard_normal((b, t, h, d)).astype(np.float32)
    thd = o.rope_thd(src4, cos, sin, b, t, h, d).reshape(b, t, h, d)
    bhtd = o.rope(np.ascontiguousarray(src4.transpose(0, 2, 1, 3)), cos, sin, b * h, t * d, d).reshape(b, h, t, d)
    assert np.array_equal(thd, bhtd.transpose(0, 2, 1, 3))
    thd2 = o.rope_thd(src4, cos2, sin2, b, t, h, d, stride_b=t * h * d).reshape(b, t, h, d)
    for i in range(b):
        assert np.array_equal(thd2[i], o.rope_thd(src4[i], cos2[i], sin2[i], 1, t, h, d).reshape(t, h, d))


def test_softmax_reference_vectors(golden):
    for c in golden["fast_softmax_f32"]:
        got = o.fast_softmax(c["src"], c["dims"][-1])
        assert _close(got, c["want"], golden["tolerance"]), c["name"]


def test_argmax_reference_vectors(golden):
    for c in golden["fast_argmax_f32"]:
        got = o.fast_argmax(c["src"], c["dims"][-1]) if c["src"] else np.zeros(0, np.uint32)
        assert list(got) == c["want"], c["name"]


def test_silu_closed_form(golden):
    for c in golden["silu_f32"]:
        want = [np.float32(x / (1 + math.exp(-x))) for x in c["inp"]]
        assert _close(o.silu(c["inp"]), want, golden["tolerance"]), c["name"]
    x = np.linspace(-20, 20, 101).astype(np.float32)
    assert _close(o.silu(x), x.astype(np.float64) / (1 + np.exp(-x.astype(np.float64))), 1e-6)


def test_index_select_is_numpy_take():
    rng = np.random.default_rng(2)
    table = rng.standard_normal((11, 6)).astype(np.float32)
    ids = np.array([3, 0, 10, 3], np.int64)
    assert np.array_equal(o.index_select(ids, table, 1, 11, 6).reshape(4, 6), table[ids])


def test_add_mul():
    a = np.array([1.5, -2, 3], np.float32)
    b = np.array([0.25, 4, -1], np.float32)
    assert np.array_equal(o.add(a, b), a + b) and np.array_equal(o.mul(a, b), a * b)


def test_attention_decode_against_float64():
    rng = np.random.default_rng(3)
    n_heads, n_kv, hd, n_pos = 8, 2, 16, 37
    q = rng.standard_normal((n_heads, hd)).astype(np.float32)
    k = rng.standard_normal((n_kv, n_pos + 3, hd)).astype(np.float32)  # cache has spare capacity
    v = rng.standard_normal((n_kv, n_pos + 3, hd)).astype(np.float32)
    scale = 1 / math.sqrt(hd)
    got = o.attention_decode(q, k, v, n_heads, n_kv, hd, n_pos, (n_pos + 3) * hd, scale).reshape(n_heads, hd)
    for h in range(n_heads):
        kk, vv = k[h // 4, :n_pos].astype(np.float64), v[h // 4, :n_pos].astype(np.float64)
        s = kk @ q[h].astype(np.float64) * scale
        p = np.exp(s - s.max())
        p /= p.sum()
        assert _close(got[h], p @ vv, 1e-5)
