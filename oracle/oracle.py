"""ctypes front end of the CPU oracle (libcandy_oracle.so).

TEST INFRASTRUCTURE ONLY. Only tests, the smoke check and the benchmark's CPU-baseline
leg may import this module; the shipped library and its host wrappers never do.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcandy_oracle.so")

Q4_0, Q8_0, Q4_K, Q6_K, Q4_0_GGML = 2, 8, 12, 14, 102
FORMATS = {"q4_0": Q4_0, "q8_0": Q8_0, "q4_k": Q4_K, "q6_k": Q6_K, "q4_0_ggml": Q4_0_GGML}


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (a few hundred ms)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        i64, vp, f32 = ctypes.c_int64, ctypes.c_void_p, ctypes.c_float
        L.co_block_elems.argtypes = [ctypes.c_int]
        L.co_block_bytes.argtypes = [ctypes.c_int]
        L.co_fp16_to_f32.argtypes = [ctypes.c_uint16]
        L.co_fp16_to_f32.restype = f32
        L.co_f32_to_fp16.argtypes = [f32]
        L.co_f32_to_fp16.restype = ctypes.c_uint16
        L.co_get_scale_min_k4.argtypes = [ctypes.c_int, vp, vp, vp]
        L.co_get_scale_min_k4.restype = None
        L.co_dequantize.argtypes = [ctypes.c_int, vp, i64, vp]
        L.co_quantize_q8_0.argtypes = [vp, i64, i64, vp]
        L.co_quantize.argtypes = [ctypes.c_int, vp, i64, i64, vp]
        L.co_quantize.restype = ctypes.c_int
        L.co_vec_dot_q8_0.argtypes = [ctypes.c_int, vp, vp, i64]
        L.co_vec_dot_q8_0.restype = f32
        L.co_make_qkx2_quants.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp, vp, vp, f32, f32, ctypes.c_int]
        L.co_make_qkx2_quants.restype = f32
        L.co_make_qx_quants.argtypes = [ctypes.c_int, ctypes.c_int, vp, vp]
        L.co_make_qx_quants.restype = f32
        L.co_set_block_order.argtypes = [ctypes.c_int]
        L.co_set_block_order.restype = None
        L.co_qmatmul.argtypes = [ctypes.c_int, vp, i64, i64, vp, i64, vp]
        L.co_matmul_dequant_f32.argtypes = [ctypes.c_int, vp, i64, i64, vp, i64, vp]
        L.co_naive_batched_matmul_f32.argtypes = [i64, i64, i64, i64, vp, vp, vp]
        L.co_naive_batched_matmul_f32.restype = None
        L.co_naive_batched_matmul_strided_f32.argtypes = [i64, i64, i64, i64, vp, vp, vp, vp, vp, vp]
        L.co_naive_batched_matmul_strided_f32.restype = None
        L.co_fast_rms_norm_f32.argtypes = [i64, i64, f32, vp, vp, vp]
        L.co_fast_rms_norm_f32.restype = None
        L.co_rope_f32.argtypes = [i64, i64, i64, i64, vp, vp, vp, vp]
        L.co_rope_f32.restype = None
        L.co_rope_i_f32.argtypes = [i64, i64, i64, vp, vp, vp, vp]
        L.co_rope_i_f32.restype = None
        L.co_rope_thd_f32.argtypes = [i64, i64, i64, i64, i64, vp, vp, vp, vp]
        L.co_rope_thd_f32.restype = None
        L.co_fast_softmax_f32.argtypes = [i64, i64, vp, vp]
        L.co_fast_softmax_f32.restype = None
        L.co_silu_f32.argtypes = [i64, vp, vp]
        L.co_silu_f32.restype = None
        L.co_fast_argmax_f32.argtypes = [i64, i64, vp, vp]
        L.co_fast_argmax_f32.restype = None
        L.co_index_select_f32.argtypes = [i64, vp, vp, vp, i64, i64, i64, i64]
        L.co_index_select_f32.restype = None
        L.co_add_f32.argtypes = [i64, vp, vp, vp]
        L.co_add_f32.restype = None
        L.co_mul_f32.argtypes = [i64, vp, vp, vp]
        L.co_mul_f32.restype = None
        L.co_attention_decode_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, f32, vp]
        L.co_attention_decode_f32.restype = None
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    return a.view(np.uint8).reshape(-1)


def block_elems(fmt: int) -> int:
    return lib().co_block_elems(fmt)


def block_bytes(fmt: int) -> int:
    return lib().co_block_bytes(fmt)


def fp16_to_f32(h: int) -> float:
    return lib().co_fp16_to_f32(int(h))


def f32_to_fp16(f: float) -> int:
    return lib().co_f32_to_fp16(float(f))


def get_scale_min_k4(j: int, scales12) -> tuple[int, int]:
    q = _u8(np.asarray(scales12, dtype=np.uint8))
    sc = np.zeros(1, np.uint8)
    m = np.zeros(1, np.uint8)
    lib().co_get_scale_min_k4(j, _p(q), _p(sc), _p(m))
    return int(sc[0]), int(m[0])


def dequantize(fmt: int, blocks) -> np.ndarray:
    b = _u8(blocks)
    bs, qk = block_bytes(fmt), block_elems(fmt)
    assert bs and b.size % bs == 0, "byte count is not a whole number of blocks"
    nb = b.size // bs
    y = np.empty(nb * qk, np.float32)
    rc = lib().co_dequantize(fmt, _p(b), nb, _p(y))
    assert rc == 0
    return y


def dequantize_f16(fmt: int, blocks) -> np.ndarray:
    """dequantize_block_*_f16 (tensor/internal/cuda/kernels/kernels.go:486-505): the kernels of the f32 output with
    dst_t = half (template quantized.cu:1229-1249 `y[...] = v.x`, and the K-quant kernels' `y[l] = d * q - m`), i.e.
    each f32 value converted on the store, which is round to nearest even."""
    return dequantize(fmt, blocks).astype(np.float16)


def dequantize_f64(fmt: int, blocks) -> np.ndarray:
    """DequantizeBlockQ4_0F64 / Q4_1F64 / Q8_0F64 (tensor/internal/cpu/kernels/quantized.go:96-104, 119-128, 139-144):
    d (and m) are the fp16 fields widened to f32 and then to f64, the arithmetic is float64."""
    b = _u8(blocks)
    if fmt == Q4_0:
        blk = b.reshape(-1, 18)
        d = blk[:, :2].copy().view(np.float16).astype(np.float32).astype(np.float64)
        qs = blk[:, 2:]
        y = np.empty((blk.shape[0], 32), np.float64)
        y[:, 0::2] = d * ((qs & 0xF).astype(np.float64) - 8)
        y[:, 1::2] = d * ((qs >> 4).astype(np.float64) - 8)
    elif fmt == 3:  # Q4_1
        blk = b.reshape(-1, 20)
        d = blk[:, :2].copy().view(np.float16).astype(np.float32).astype(np.float64)
        m = blk[:, 2:4].copy().view(np.float16).astype(np.float32).astype(np.float64)
        qs = blk[:, 4:]
        y = np.empty((blk.shape[0], 32), np.float64)
        y[:, 0::2] = d * (qs & 0xF).astype(np.float64) + m
        y[:, 1::2] = d * (qs >> 4).astype(np.float64) + m
    elif fmt == Q8_0:
        blk = b.reshape(-1, 34)
        d = blk[:, :2].copy().view(np.float16).astype(np.float32).astype(np.float64)
        y = d * blk[:, 2:].copy().view(np.int8).astype(np.float64)
    else:
        raise ValueError(f"no float64 dequantize for format {fmt}")
    return y.reshape(-1)


def quantize_q8_0(x, rows: int | None = None, cols: int | None = None) -> np.ndarray:
    x = _f32(x)
    if rows is None:
        x2 = x.reshape(-1, x.shape[-1]) if x.ndim > 1 else x.reshape(1, -1)
        rows, cols = x2.shape
    out = np.empty(rows * cols // 32 * 34, np.uint8)
    rc = lib().co_quantize_q8_0(_p(x), rows, cols, _p(out))
    assert rc == 0, "cols must be a multiple of 32"
    return out


def quantize(fmt: int, x, rows: int | None = None, cols: int | None = None) -> np.ndarray:
    """f32 [rows, cols] -> blocks of fmt (ggml's reference quantizers; parity unpinned, see candy_oracle.c)."""
    x = _f32(x)
    if rows is None:
        x2 = x.reshape(-1, x.shape[-1]) if x.ndim > 1 else x.reshape(1, -1)
        rows, cols = x2.shape
    qk = block_elems(fmt)
    assert qk and cols % qk == 0, "cols must be a multiple of the block"
    out = np.empty(rows * cols // qk * block_bytes(fmt), np.uint8)
    rc = lib().co_quantize(fmt, _p(x), rows, cols, _p(out))
    assert rc == 0
    return out


def make_qkx2_quants(x, weights, nmax=15, rmin=-1.0, rdelta=0.1, nstep=20):
    """Test hook: (scale, -min, levels) of the Q4_K sub-block search."""
    x, weights = _f32(x).reshape(-1), _f32(weights).reshape(-1)
    L = np.zeros(x.size, np.uint8)
    the_min = np.zeros(1, np.float32)
    scale = lib().co_make_qkx2_quants(x.size, nmax, _p(x), _p(weights), _p(L), _p(the_min), rmin, rdelta, nstep)
    return float(scale), float(the_min[0]), L


def make_qx_quants(x, nmax=32):
    """Test hook: (scale, levels + nmax) of the Q6_K group search."""
    x = _f32(x).reshape(-1)
    L = np.zeros(x.size, np.int8)
    scale = lib().co_make_qx_quants(x.size, nmax, _p(x), _p(L))
    return float(scale), L


def vec_dot_q8_0(fmt: int, w_row, x_q8_0, k: int) -> float:
    return lib().co_vec_dot_q8_0(fmt, _p(_u8(w_row)), _p(_u8(x_q8_0)), k)


def set_block_order(order: int):
    """Test aid: the order vec-dots add a row's blocks in (0 ascending, 1 descending, 2 even then odd, 3 second
    half first); process-wide."""
    lib().co_set_block_order(int(order))


def qmatmul(fmt: int, w_blocks, rows: int, cols: int, x) -> np.ndarray:
    x = _f32(x).reshape(-1, cols)
    m = x.shape[0]
    w = _u8(w_blocks)
    assert w.size == rows * cols // block_elems(fmt) * block_bytes(fmt)
    y = np.empty((m, rows), np.float32)
    rc = lib().co_qmatmul(fmt, _p(w), rows, cols, _p(x), m, _p(y))
    assert rc == 0
    return y


def matmul_dequant_f32(fmt: int, w_blocks, rows: int, cols: int, x) -> np.ndarray:
    x = _f32(x).reshape(-1, cols)
    m = x.shape[0]
    w = _u8(w_blocks)
    y = np.empty((m, rows), np.float32)
    rc = lib().co_matmul_dequant_f32(fmt, _p(w), rows, cols, _p(x), m, _p(y))
    assert rc == 0
    return y


def naive_batched_matmul_f32(b, m, n, k, a, bm) -> np.ndarray:
    a, bm = _f32(a), _f32(bm)
    c = np.empty(b * m * n, np.float32)
    lib().co_naive_batched_matmul_f32(b, m, n, k, _p(a), _p(bm), _p(c))
    return c


def naive_batched_matmul_strided_f32(b, m, n, k, a, bm, a_strides, b_strides, c_strides, c_size) -> np.ndarray:
    a, bm = _f32(a), _f32(bm)
    c = np.zeros(c_size, np.float32)
    s = [np.asarray(v, np.int64) for v in (a_strides, b_strides, c_strides)]
    lib().co_naive_batched_matmul_strided_f32(b, m, n, k, _p(a), _p(bm), _p(c), _p(s[0]), _p(s[1]), _p(s[2]))
    return c


def fast_rms_norm(x, ncols: int, eps: float, alpha=None) -> np.ndarray:
    x = _f32(x).reshape(-1)
    dst = np.empty_like(x)
    al = _f32(alpha) if alpha is not None else None
    lib().co_fast_rms_norm_f32(x.size, ncols, eps, _p(al) if al is not None else None, _p(x), _p(dst))
    return dst


def rope(src, cos, sin, bh: int, td: int, d: int, stride_b: int = 0) -> np.ndarray:
    src, cos, sin = _f32(src).reshape(-1), _f32(cos).reshape(-1), _f32(sin).reshape(-1)
    dst = src.copy()
    lib().co_rope_f32(bh, td, d, stride_b, _p(src), _p(cos), _p(sin), _p(dst))
    return dst


def rope_i(src, cos, sin, bh: int, td: int, stride_b: int = 0) -> np.ndarray:
    """RopeIF32 (reduce.go:3825-3838): adjacent pairs."""
    src, cos, sin = _f32(src).reshape(-1), _f32(cos).reshape(-1), _f32(sin).reshape(-1)
    dst = src.copy()
    lib().co_rope_i_f32(bh, td, stride_b, _p(src), _p(cos), _p(sin), _p(dst))
    return dst


def rope_thd(src, cos, sin, b: int, t: int, h: int, d: int, stride_b: int = 0) -> np.ndarray:
    """RopeThdF32 (reduce.go:4178-4196): [b, t, h, d] layout, half-split pairs."""
    src, cos, sin = _f32(src).reshape(-1), _f32(cos).reshape(-1), _f32(sin).reshape(-1)
    dst = src.copy()
    lib().co_rope_thd_f32(b, t, h, d, stride_b, _p(src), _p(cos), _p(sin), _p(dst))
    return dst


def fast_softmax(src, ncols: int) -> np.ndarray:
    src = _f32(src).reshape(-1)
    dst = np.empty_like(src)
    lib().co_fast_softmax_f32(src.size, ncols, _p(src), _p(dst))
    return dst


def silu(x) -> np.ndarray:
    x = _f32(x).reshape(-1)
    out = np.empty_like(x)
    lib().co_silu_f32(x.size, _p(x), _p(out))
    return out


def fast_argmax(src, ncols: int) -> np.ndarray:
    src = _f32(src).reshape(-1)
    n = src.size // ncols if ncols else 0
    dst = np.zeros(n, np.uint32)
    lib().co_fast_argmax_f32(src.size, ncols, _p(src), _p(dst))
    return dst


def index_select(ids, inp, left: int, src_dim: int, right: int) -> np.ndarray:
    ids = np.ascontiguousarray(ids, np.int64)
    inp = _f32(inp).reshape(-1)
    out = np.empty(left * ids.size * right, np.float32)
    lib().co_index_select_f32(out.size, _p(ids), _p(inp), _p(out), left, src_dim, ids.size, right)
    return out


def add(a, b) -> np.ndarray:
    a, b = _f32(a).reshape(-1), _f32(b).reshape(-1)
    out = np.empty_like(a)
    lib().co_add_f32(a.size, _p(a), _p(b), _p(out))
    return out


def mul(a, b) -> np.ndarray:
    a, b = _f32(a).reshape(-1), _f32(b).reshape(-1)
    out = np.empty_like(a)
    lib().co_mul_f32(a.size, _p(a), _p(b), _p(out))
    return out


def attention_decode(q, k_cache, v_cache, n_heads, n_kv_heads, head_dim, n_pos, cache_stride, scale) -> np.ndarray:
    q, k_cache, v_cache = _f32(q).reshape(-1), _f32(k_cache).reshape(-1), _f32(v_cache).reshape(-1)
    out = np.empty(n_heads * head_dim, np.float32)
    lib().co_attention_decode_f32(_p(q), _p(k_cache), _p(v_cache), n_heads, n_kv_heads, head_dim,
                                  n_pos, cache_stride, scale, _p(out))
    return out
