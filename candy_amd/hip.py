"""ctypes binding of libcandy_hip.so (include/candy_hip.h).

There is no CPU fallback: importing works anywhere (so the symbol table can be checked
without a GPU), but every compute call goes to the HIP library and raises CandyHipError
when the library or the GPU is missing.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, byref, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint32, c_void_p

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcandy_hip.so")

Q4_0, Q8_0, Q4_K, Q6_K, Q4_0_GGML = 2, 8, 12, 14, 102

W_ATTN_NORM, W_Q, W_K, W_V, W_O, W_FFN_NORM, W_GATE, W_UP, W_DOWN, W_OUT_NORM, W_HEAD, W_EMBED = range(12)


class CandyHipError(RuntimeError):
    def __init__(self, status: int, text: str):
        super().__init__(f"candy_hip status {status}: {text}")
        self.status = status
        self.text = text


class LlamaConfig(ctypes.Structure):
    _fields_ = [("n_layers", c_int32), ("d_model", c_int32), ("n_heads", c_int32), ("n_kv_heads", c_int32),
                ("head_dim", c_int32), ("d_ffn", c_int32), ("vocab", c_int32), ("max_pos", c_int32),
                ("rms_eps", c_float), ("rope_base", c_float)]


# name -> (restype, argtypes); exactly the symbols include/candy_hip.h declares
SIGNATURES = {
    "candy_hip_last_error": (c_char_p, []),
    "candy_hip_version": (c_char_p, []),
    "candy_hip_device_count": (c_int, [POINTER(c_int)]),
    "candy_hip_open": (c_int, [c_int, POINTER(c_void_p)]),
    "candy_hip_close": (c_int, [c_void_p]),
    "candy_hip_device_ordinal": (c_int, [c_void_p, POINTER(c_int)]),
    "candy_hip_device_name": (c_int, [c_void_p, c_char_p, c_size_t]),
    "candy_hip_synchronize": (c_int, [c_void_p]),
    "candy_hip_set_option": (c_int, [c_void_p, c_char_p, c_int64]),
    "candy_hip_get_option": (c_int, [c_void_p, c_char_p, POINTER(c_int64)]),
    "candy_hip_alloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "candy_hip_free": (c_int, [c_void_p, c_void_p]),
    "candy_hip_zero": (c_int, [c_void_p, c_void_p, c_size_t]),
    "candy_hip_h2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "candy_hip_d2h": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "candy_hip_d2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "candy_hip_block_elems": (c_int, [c_int]),
    "candy_hip_block_bytes": (c_int, [c_int]),
    "candy_hip_qweight_bytes": (c_size_t, [c_int, c_int64, c_int64]),
    "candy_hip_qtensor_upload": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_size_t, POINTER(c_void_p)]),
    "candy_hip_qtensor_wrap": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_size_t, POINTER(c_void_p)]),
    "candy_hip_qtensor_free": (c_int, [c_void_p]),
    "candy_hip_qtensor_info": (c_int, [c_void_p, POINTER(c_int), POINTER(c_int64), POINTER(c_int64),
                                       POINTER(c_size_t), POINTER(c_void_p)]),
    "candy_hip_dequantize_blocks": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "candy_hip_dequantize": (c_int, [c_void_p, c_void_p, c_void_p]),
    "candy_hip_dequantize_blocks_f16": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "candy_hip_dequantize_f16": (c_int, [c_void_p, c_void_p, c_void_p]),
    "candy_hip_dequantize_blocks_f64": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_void_p]),
    "candy_hip_dmmv": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "candy_hip_quantize_q8_0": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "candy_hip_quantize": (c_int, [c_void_p, c_int, c_void_p, c_int64, c_int64, c_void_p]),
    "candy_hip_qmatmul": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_qmatmul_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_qmatmul_q8": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_qact_create": (c_int, [c_void_p, c_int64, c_int64, POINTER(c_void_p)]),
    "candy_hip_qact_free": (c_int, [c_void_p]),
    "candy_hip_qact_quantize": (c_int, [c_void_p, c_void_p, c_int64, c_int64]),
    "candy_hip_qmatmul_qact": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p]),
    "candy_hip_matmul_f32": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int]),
    "candy_hip_matmul_f32_strided": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                             c_int64, c_int64, c_int64]),
    "candy_hip_rms_norm": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int64, c_void_p]),
    "candy_hip_rope": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_void_p]),
    "candy_hip_rope_i": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "candy_hip_rope_thd": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64, c_int64,
                                   c_void_p]),
    "candy_hip_softmax": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "candy_hip_silu": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_add": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_silu_mul": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_argmax": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p]),
    "candy_hip_index_select": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_void_p]),
    "candy_hip_qindex_select": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "candy_hip_attention_decode": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int64,
                                           c_int64, c_float, c_void_p]),
    "candy_hip_llama_create": (c_int, [c_void_p, POINTER(LlamaConfig), POINTER(c_void_p)]),
    "candy_hip_llama_free": (c_int, [c_void_p]),
    "candy_hip_llama_set_qweight": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "candy_hip_llama_set_norm": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "candy_hip_llama_set_graph": (c_int, [c_void_p, c_int]),
    "candy_hip_llama_set_kv_f16": (c_int, [c_void_p, c_int]),
    "candy_hip_llama_kv_cache": (c_int, [c_void_p, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_size_t)]),
    "candy_hip_llama_hidden": (c_int, [c_void_p, POINTER(c_void_p)]),
    "candy_hip_llama_decode": (c_int, [c_void_p, c_int32, c_int32, POINTER(c_void_p), POINTER(c_int32)]),
    "candy_hip_llama_generate": (c_int, [c_void_p, c_int32, c_int32, c_int32, POINTER(c_int32)]),
    "candy_hip_llama_decode_hidden": (c_int, [c_void_p, c_void_p, c_int32, POINTER(c_void_p), POINTER(c_int32)]),
    "candy_hip_llama_prefill": (c_int, [c_void_p, POINTER(c_int32), c_int32, c_int32, POINTER(c_void_p),
                                        POINTER(c_int32)]),
    "candy_hip_qmatmul_sweep": (c_int, [c_void_p, POINTER(c_void_p), c_int, c_void_p, c_int64, c_void_p, c_int, c_int,
                                        POINTER(c_float)]),
    "candy_hip_qmatmul_sustained_sweep": (c_int, [c_void_p, POINTER(c_void_p), c_int, c_int, c_int, c_void_p, c_void_p, c_int,
                                                  POINTER(c_float)]),
    "candy_hip_dequantize_sweep": (c_int, [c_void_p, POINTER(c_void_p), c_int, c_void_p, c_int, c_int, POINTER(c_float)]),
    "candy_hip_quantize_sweep": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int64, c_int64, c_void_p, c_int, c_int,
                                         POINTER(c_float)]),
    "candy_hip_stream_probe": (c_int, [c_void_p, c_size_t, c_size_t, c_int, POINTER(c_float)]),
    "candy_hip_launch_probe": (c_int, [c_void_p, c_int, c_int, POINTER(c_float)]),
    "candy_hip_timer_start": (c_int, [c_void_p]),
    "candy_hip_timer_stop": (c_int, [c_void_p, POINTER(c_float)]),
}

_lib = None


def lib() -> ctypes.CDLL:
    """Load libcandy_hip.so; raises if it has not been built (there is nothing to fall back to)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise CandyHipError(-1, f"{LIB_PATH} is missing: build it with `make -C candy_amd/csrc` "
                                    "(or __graft_entry__.build())")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def _check(status: int):
    if status != 0:
        raise CandyHipError(status, lib().candy_hip_last_error().decode(errors="replace"))


def device_count() -> int:
    n = c_int(0)
    rc = lib().candy_hip_device_count(byref(n))
    return n.value if rc == 0 else 0


class Buffer:
    """A raw device allocation (what backs a BackendStorage)."""

    def __init__(self, dev: "Device", nbytes: int):
        self.dev, self.nbytes = dev, int(nbytes)
        p = c_void_p()
        _check(lib().candy_hip_alloc(dev.handle, self.nbytes, byref(p)))
        self.ptr = p.value

    def free(self):
        if self.ptr is not None and self.dev.handle is not None:
            _check(lib().candy_hip_free(self.dev.handle, self.ptr))
        self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def upload(self, arr: np.ndarray, offset: int = 0) -> "Buffer":
        a = np.ascontiguousarray(arr)
        assert offset + a.nbytes <= self.nbytes
        _check(lib().candy_hip_h2d(self.dev.handle, self.ptr + offset, a.ctypes.data, a.nbytes))
        return self

    def download(self, dtype, count: int | None = None, offset: int = 0) -> np.ndarray:
        dt = np.dtype(dtype)
        if count is None:
            count = (self.nbytes - offset) // dt.itemsize
        out = np.empty(count, dt)
        _check(lib().candy_hip_d2h(self.dev.handle, out.ctypes.data, self.ptr + offset, out.nbytes))
        return out

    def zero(self) -> "Buffer":
        _check(lib().candy_hip_zero(self.dev.handle, self.ptr, self.nbytes))
        return self


class QTensor:
    """Device-resident quantized weight [rows, cols] in its original block layout."""

    def __init__(self, dev: "Device", fmt: int, rows: int, cols: int, blocks: np.ndarray):
        b = np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)
        h = c_void_p()
        _check(lib().candy_hip_qtensor_upload(dev.handle, fmt, rows, cols, b.ctypes.data, b.nbytes, byref(h)))
        self.dev, self.fmt, self.rows, self.cols, self.nbytes, self.handle = dev, fmt, rows, cols, b.nbytes, h.value

    @classmethod
    def quantize(cls, dev: "Device", fmt: int, x: np.ndarray) -> "QTensor":
        """f32 [rows, cols] -> a weight of format fmt, quantized on the device and kept there."""
        x = np.ascontiguousarray(x, np.float32)
        rows, cols = x.reshape(-1, x.shape[-1]).shape
        nbytes = lib().candy_hip_qweight_bytes(fmt, rows, cols)
        src = dev.from_numpy(x)
        dst = dev.alloc(nbytes + 64)  # spare bytes after the blocks: every tile kernel may take the weight
        _check(lib().candy_hip_quantize(dev.handle, fmt, src.ptr, rows, cols, dst.ptr))
        q = cls.__new__(cls)
        h = c_void_p()
        _check(lib().candy_hip_qtensor_wrap(dev.handle, fmt, rows, cols, dst.ptr, nbytes + 64, byref(h)))
        q.dev, q.fmt, q.rows, q.cols, q.nbytes, q.handle = dev, fmt, rows, cols, nbytes, h.value
        q._blocks = dst  # the wrapped device memory stays owned here
        return q

    def free(self):
        if self.handle is not None and self.dev.handle is not None:
            _check(lib().candy_hip_qtensor_free(self.handle))
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Device:
    """One GPU: candy.BackendDevice on the HIP side."""

    def __init__(self, ordinal: int = 0):
        h = c_void_p()
        _check(lib().candy_hip_open(ordinal, byref(h)))
        self.handle = h.value
        buf = ctypes.create_string_buffer(256)
        _check(lib().candy_hip_device_name(self.handle, buf, 256))
        self.name = buf.value.decode()

    def close(self):
        if self.handle is not None:
            lib().candy_hip_close(self.handle)
            self.handle = None

    # ---- switches (include/candy_hip.h lists the keys)
    def set_option(self, key: str, value: int):
        _check(lib().candy_hip_set_option(self.handle, key.encode(), int(value)))

    def get_option(self, key: str) -> int:
        v = c_int64(0)
        _check(lib().candy_hip_get_option(self.handle, key.encode(), byref(v)))
        return v.value

    # ---- memory
    def alloc(self, nbytes: int) -> Buffer:
        return Buffer(self, nbytes)

    def from_numpy(self, arr: np.ndarray) -> Buffer:
        a = np.ascontiguousarray(arr)
        return Buffer(self, max(a.nbytes, 1)).upload(a) if a.nbytes else Buffer(self, 1)

    def synchronize(self):
        _check(lib().candy_hip_synchronize(self.handle))

    def qtensor(self, fmt: int, rows: int, cols: int, blocks: np.ndarray) -> QTensor:
        return QTensor(self, fmt, rows, cols, blocks)

    # ---- quantized path
    def dequantize_blocks(self, fmt: int, blocks: np.ndarray) -> np.ndarray:
        b = np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)
        bs, qk = lib().candy_hip_block_bytes(fmt), lib().candy_hip_block_elems(fmt)
        if bs == 0:
            _check(lib().candy_hip_dequantize_blocks(self.handle, fmt, None, 0, None))
        nb = b.size // bs
        src = self.from_numpy(b)
        dst = self.alloc(max(nb * qk * 4, 16))
        _check(lib().candy_hip_dequantize_blocks(self.handle, fmt, src.ptr, nb, dst.ptr))
        return dst.download(np.float32, nb * qk)

    def dequantize(self, q: QTensor) -> np.ndarray:
        dst = self.alloc(q.rows * q.cols * 4)
        _check(lib().candy_hip_dequantize(self.handle, q.handle, dst.ptr))
        return dst.download(np.float32, q.rows * q.cols).reshape(q.rows, q.cols)

    def dequantize_blocks_as(self, fmt: int, blocks: np.ndarray, dtype) -> np.ndarray:
        """Blocks -> float16 or float64 values (the reference's other dequantize outputs)."""
        dtype = np.dtype(dtype)
        entry = {np.dtype(np.float16): lib().candy_hip_dequantize_blocks_f16,
                 np.dtype(np.float64): lib().candy_hip_dequantize_blocks_f64}[dtype]
        b = np.ascontiguousarray(blocks).view(np.uint8).reshape(-1)
        bs, qk = lib().candy_hip_block_bytes(fmt), lib().candy_hip_block_elems(fmt)
        if bs == 0:
            _check(entry(self.handle, fmt, None, 0, None))
        nb = b.size // bs
        src = self.from_numpy(b)
        dst = self.alloc(max(nb * qk * dtype.itemsize, 16))
        _check(entry(self.handle, fmt, src.ptr, nb, dst.ptr))
        return dst.download(dtype, nb * qk)

    def dequantize_f16(self, q: QTensor) -> np.ndarray:
        dst = self.alloc(q.rows * q.cols * 2)
        _check(lib().candy_hip_dequantize_f16(self.handle, q.handle, dst.ptr))
        return dst.download(np.float16, q.rows * q.cols).reshape(q.rows, q.cols)

    def dmmv(self, q: QTensor, x: np.ndarray) -> np.ndarray:
        """y[rows] = dequantize(W) . x with f32 activations (no activation quantizer)."""
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        assert x.size == q.cols
        src = self.from_numpy(x)
        dst = self.alloc(max(q.rows * 4, 16))
        _check(lib().candy_hip_dmmv(self.handle, q.handle, src.ptr, dst.ptr))
        return dst.download(np.float32, q.rows)

    def quantize_q8_0(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32)
        x2 = x.reshape(-1, x.shape[-1]) if x.ndim > 1 else x.reshape(1, -1)
        rows, cols = x2.shape
        src = self.from_numpy(x2)
        dst = self.alloc(max(rows * cols // 32 * 34, 2))
        _check(lib().candy_hip_quantize_q8_0(self.handle, src.ptr, rows, cols, dst.ptr))
        return dst.download(np.uint8, rows * cols // 32 * 34)

    def quantize(self, fmt: int, x: np.ndarray) -> np.ndarray:
        """f32 [rows, cols] -> the blocks of format fmt (host bytes), quantized on the device."""
        x = np.ascontiguousarray(x, np.float32)
        x2 = x.reshape(-1, x.shape[-1]) if x.ndim > 1 else x.reshape(1, -1)
        rows, cols = x2.shape
        nbytes = lib().candy_hip_qweight_bytes(fmt, rows, cols)
        src = self.from_numpy(x2)
        dst = self.alloc(max(nbytes, 2))
        _check(lib().candy_hip_quantize(self.handle, fmt, src.ptr, rows, cols, dst.ptr))
        return dst.download(np.uint8, nbytes)

    def qmatmul(self, w: QTensor, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32).reshape(-1, w.cols)
        m = x.shape[0]
        src = self.from_numpy(x)
        dst = self.alloc(max(m * w.rows * 4, 4))
        _check(lib().candy_hip_qmatmul(self.handle, w.handle, src.ptr, m, dst.ptr))
        return dst.download(np.float32, m * w.rows).reshape(m, w.rows)

    def qmatmul_q8(self, w: QTensor, x_blocks: np.ndarray, m: int) -> np.ndarray:
        src = self.from_numpy(np.ascontiguousarray(x_blocks).view(np.uint8))
        dst = self.alloc(max(m * w.rows * 4, 4))
        _check(lib().candy_hip_qmatmul_q8(self.handle, w.handle, src.ptr, m, dst.ptr))
        return dst.download(np.float32, m * w.rows).reshape(m, w.rows)

    # ---- f32 ops (host arrays in, host arrays out; the C ABI itself works on device pointers)
    def _f32(self, a) -> Buffer:
        return self.from_numpy(np.ascontiguousarray(a, np.float32).reshape(-1))

    def matmul_f32(self, a, b, batch, m, n, k, rhs_transposed=False) -> np.ndarray:
        da, db = self._f32(a), self._f32(b)
        dc = self.alloc(max(batch * m * n * 4, 4))
        _check(lib().candy_hip_matmul_f32(self.handle, da.ptr, db.ptr, dc.ptr, batch, m, n, k, int(rhs_transposed)))
        return dc.download(np.float32, batch * m * n)

    def matmul_f32_strided(self, a, b, m, n, k, a_strides, b_strides, a_offset=0, b_offset=0) -> np.ndarray:
        """One batch; a_strides / b_strides are (row, column) element strides, the offsets the layouts' start offsets."""
        da, db = self._f32(a), self._f32(b)
        dc = self.alloc(m * n * 4)
        _check(lib().candy_hip_matmul_f32_strided(self.handle, da.ptr + 4 * a_offset, db.ptr + 4 * b_offset, dc.ptr, m, n, k,
                                                  a_strides[0], a_strides[1], b_strides[0], b_strides[1]))
        return dc.download(np.float32, m * n)

    def rms_norm(self, x, cols: int, eps: float, alpha=None) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        rows = x.size // cols if cols else 0
        dx = self._f32(x)
        da = self._f32(alpha) if alpha is not None else None
        out = self.alloc(max(x.nbytes, 4))
        _check(lib().candy_hip_rms_norm(self.handle, dx.ptr, da.ptr if da else None, eps, rows, cols, out.ptr))
        return out.download(np.float32, x.size)

    def rope(self, src, cos, sin, bh, td, d, stride_b=0) -> np.ndarray:
        src = np.ascontiguousarray(src, np.float32).reshape(-1)
        ds, dc, dn = self._f32(src), self._f32(cos), self._f32(sin)
        out = self.from_numpy(src)
        _check(lib().candy_hip_rope(self.handle, ds.ptr, dc.ptr, dn.ptr, bh, td, d, stride_b, out.ptr))
        return out.download(np.float32, src.size)

    def rope_i(self, src, cos, sin, bh, td, stride_b=0) -> np.ndarray:
        """RopeI (backend.go:156): adjacent pairs."""
        src = np.ascontiguousarray(src, np.float32).reshape(-1)
        if src.size == 0:
            return src.copy()
        ds, dc, dn = self._f32(src), self._f32(cos), self._f32(sin)
        out = self.from_numpy(src)
        _check(lib().candy_hip_rope_i(self.handle, ds.ptr, dc.ptr, dn.ptr, bh, td, stride_b, out.ptr))
        return out.download(np.float32, src.size)

    def rope_thd(self, src, cos, sin, b, t, h, d, stride_b=0) -> np.ndarray:
        """RopeThd (backend.go:162): [b, t, h, d] layout."""
        src = np.ascontiguousarray(src, np.float32).reshape(-1)
        if src.size == 0:
            return src.copy()
        ds, dc, dn = self._f32(src), self._f32(cos), self._f32(sin)
        out = self.from_numpy(src)
        _check(lib().candy_hip_rope_thd(self.handle, ds.ptr, dc.ptr, dn.ptr, b, t, h, d, stride_b, out.ptr))
        return out.download(np.float32, src.size)

    def softmax(self, src, cols: int) -> np.ndarray:
        src = np.ascontiguousarray(src, np.float32).reshape(-1)
        rows = src.size // cols if cols else 0
        ds = self._f32(src)
        out = self.alloc(max(src.nbytes, 4))
        _check(lib().candy_hip_softmax(self.handle, ds.ptr, rows, cols, out.ptr))
        return out.download(np.float32, src.size)

    def _binary(self, fn, a, b) -> np.ndarray:
        a = np.ascontiguousarray(a, np.float32).reshape(-1)
        da, db = self._f32(a), self._f32(b)
        out = self.alloc(max(a.nbytes, 4))
        _check(fn(self.handle, da.ptr, db.ptr, a.size, out.ptr))
        return out.download(np.float32, a.size)

    def add(self, a, b):
        return self._binary(lib().candy_hip_add, a, b)

    def mul(self, a, b):
        return self._binary(lib().candy_hip_mul, a, b)

    def silu_mul(self, gate, up):
        return self._binary(lib().candy_hip_silu_mul, gate, up)

    def silu(self, x) -> np.ndarray:
        x = np.ascontiguousarray(x, np.float32).reshape(-1)
        dx = self._f32(x)
        out = self.alloc(max(x.nbytes, 4))
        _check(lib().candy_hip_silu(self.handle, dx.ptr, x.size, out.ptr))
        return out.download(np.float32, x.size)

    def argmax(self, src, cols: int) -> np.ndarray:
        src = np.ascontiguousarray(src, np.float32).reshape(-1)
        rows = src.size // cols if cols else 0
        ds = self._f32(src)
        out = self.alloc(max(rows * 4, 4))
        _check(lib().candy_hip_argmax(self.handle, ds.ptr, rows, cols, out.ptr))
        return out.download(np.uint32, rows)

    def index_select(self, table, ids) -> np.ndarray:
        table = np.ascontiguousarray(table, np.float32)
        ids = np.ascontiguousarray(ids, np.int64)
        dt, di = self._f32(table), self.from_numpy(ids)
        out = self.alloc(max(ids.size * table.shape[1] * 4, 4))
        _check(lib().candy_hip_index_select(self.handle, dt.ptr, table.shape[0], table.shape[1], di.ptr, ids.size, out.ptr))
        return out.download(np.float32, ids.size * table.shape[1]).reshape(ids.size, table.shape[1])

    def qindex_select(self, q: QTensor, ids) -> np.ndarray:
        ids = np.ascontiguousarray(ids, np.int64)
        di = self.from_numpy(ids)
        out = self.alloc(max(ids.size * q.cols * 4, 16))
        _check(lib().candy_hip_qindex_select(self.handle, q.handle, di.ptr, ids.size, out.ptr))
        return out.download(np.float32, ids.size * q.cols).reshape(ids.size, q.cols)

    def attention_decode(self, q, k_cache, v_cache, n_heads, n_kv_heads, head_dim, n_pos, cache_stride, scale):
        dq, dk, dv = self._f32(q), self._f32(k_cache), self._f32(v_cache)
        out = self.alloc(n_heads * head_dim * 4)
        _check(lib().candy_hip_attention_decode(self.handle, dq.ptr, dk.ptr, dv.ptr, n_heads, n_kv_heads, head_dim,
                                                n_pos, cache_stride, scale, out.ptr))
        return out.download(np.float32, n_heads * head_dim)

    # ---- timing
    def qmatmul_sweep(self, weights: list, x_buf: "Buffer", m: int, y_buf: "Buffer", iters: int,
                      quantize_each: bool = True) -> float:
        """Elapsed milliseconds of `iters` back-to-back contractions rotating over `weights`."""
        arr = (c_void_p * len(weights))(*[w.handle for w in weights])
        ms = c_float(0)
        _check(lib().candy_hip_qmatmul_sweep(self.handle, arr, len(weights), x_buf.ptr, m, y_buf.ptr, iters,
                                             int(quantize_each), byref(ms)))
        return ms.value

    def qmatmul_sustained_sweep(self, weights: list, group: int, n_streams: int, x_buf: "Buffer", y_buf: "Buffer",
                                iters: int) -> float:
        """Elapsed milliseconds of `iters` batch-1 launches of `group` weights each, alternating over `n_streams`
        streams (y_buf: n_streams * group * rows floats)."""
        arr = (c_void_p * len(weights))(*[w.handle for w in weights])
        ms = c_float(0)
        _check(lib().candy_hip_qmatmul_sustained_sweep(self.handle, arr, len(weights), group, n_streams, x_buf.ptr,
                                                       y_buf.ptr, iters, byref(ms)))
        return ms.value

    def dequantize_sweep(self, weights: list, out_buf: "Buffer", iters: int, n_out: int = 1) -> float:
        """out_buf holds n_out outputs of rows*cols f32 end to end; iteration i writes output i % n_out."""
        arr = (c_void_p * len(weights))(*[w.handle for w in weights])
        ms = c_float(0)
        _check(lib().candy_hip_dequantize_sweep(self.handle, arr, len(weights), out_buf.ptr, n_out, iters, byref(ms)))
        return ms.value

    def quantize_sweep(self, x_buf: "Buffer", x_stride: int, n_x: int, rows: int, cols: int, out_buf: "Buffer",
                       iters: int, n_out: int = 1) -> float:
        ms = c_float(0)
        _check(lib().candy_hip_quantize_sweep(self.handle, x_buf.ptr, x_stride, n_x, rows, cols, out_buf.ptr, n_out,
                                              iters, byref(ms)))
        return ms.value

    def stream_probe(self, bytes_per_launch: int, span_bytes: int, iters: int) -> float:
        """Elapsed milliseconds of `iters` read-only launches (0 bytes: empty kernels)."""
        ms = c_float(0)
        _check(lib().candy_hip_stream_probe(self.handle, bytes_per_launch, span_bytes, iters, byref(ms)))
        return ms.value

    def launch_probe(self, kind: int, iters: int) -> float:
        """Elapsed milliseconds of `iters` launches of an empty kernel (kind 0: one wavefront, 1: 1024 workgroups) or
        of a kernel whose wavefronts issue one load each (2: cache-warm, 3: cold)."""
        ms = c_float(0)
        _check(lib().candy_hip_launch_probe(self.handle, kind, iters, byref(ms)))
        return ms.value

    def timer_start(self):
        _check(lib().candy_hip_timer_start(self.handle))

    def timer_stop(self) -> float:
        ms = c_float(0)
        _check(lib().candy_hip_timer_stop(self.handle, byref(ms)))
        return ms.value


class Llama:
    """Llama-style decoder on the device (weights stay owned by the caller)."""

    def __init__(self, dev: Device, **cfg):
        self.dev = dev
        self.cfg = LlamaConfig(**cfg)
        h = c_void_p()
        _check(lib().candy_hip_llama_create(dev.handle, byref(self.cfg), byref(h)))
        self.handle = h.value
        self._keep = []

    def free(self):
        if self.handle is not None and self.dev.handle is not None:
            _check(lib().candy_hip_llama_free(self.handle))
        self.handle = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass

    def set_qweight(self, which: int, layer: int, w: QTensor):
        self._keep.append(w)
        _check(lib().candy_hip_llama_set_qweight(self.handle, which, layer, w.handle))

    def set_norm(self, which: int, layer: int, alpha: np.ndarray):
        buf = self.dev.from_numpy(np.ascontiguousarray(alpha, np.float32))
        self._keep.append(buf)
        _check(lib().candy_hip_llama_set_norm(self.handle, which, layer, buf.ptr))

    def set_graph(self, enable: bool):
        _check(lib().candy_hip_llama_set_graph(self.handle, int(enable)))

    def set_kv_f16(self, enable: bool):
        """fp16 KV cache (clears the cache); kv_cache() then reports half the bytes."""
        _check(lib().candy_hip_llama_set_kv_f16(self.handle, int(enable)))

    def kv_cache(self):
        k, v, n = c_void_p(), c_void_p(), c_size_t()
        _check(lib().candy_hip_llama_kv_cache(self.handle, byref(k), byref(v), byref(n)))
        return k.value, v.value, n.value

    def hidden(self) -> np.ndarray:
        """The residual stream as the last decode step left it behind the last layer (before the final norm)."""
        p = c_void_p()
        _check(lib().candy_hip_llama_hidden(self.handle, byref(p)))
        out = np.empty(self.cfg.d_model, np.float32)
        _check(lib().candy_hip_d2h(self.dev.handle, out.ctypes.data, p.value, out.nbytes))
        return out

    def decode(self, token: int, pos: int, want_logits: bool = True):
        lg, nt = c_void_p(), c_int32(-1)
        _check(lib().candy_hip_llama_decode(self.handle, token, pos, byref(lg), byref(nt)))
        return self._result(lg, nt, want_logits)

    def generate(self, token: int, pos: int, n_steps: int):
        """n_steps greedy steps without a host round trip between them; returns the chosen tokens."""
        out = (c_int32 * n_steps)()
        _check(lib().candy_hip_llama_generate(self.handle, token, pos, n_steps, out))
        return [int(t) for t in out]

    def decode_hidden(self, hidden: np.ndarray, pos: int, want_logits: bool = True):
        buf = self.dev.from_numpy(np.ascontiguousarray(hidden, np.float32))
        lg, nt = c_void_p(), c_int32(-1)
        _check(lib().candy_hip_llama_decode_hidden(self.handle, buf.ptr, pos, byref(lg), byref(nt)))
        return self._result(lg, nt, want_logits)

    def prefill(self, tokens, pos0: int = 0, want_logits: bool = True):
        """Batched prompt pass; returns (greedy next token, logits) of the last prompt token."""
        ids = (c_int32 * len(tokens))(*[int(t) for t in tokens])
        lg, nt = c_void_p(), c_int32(-1)
        _check(lib().candy_hip_llama_prefill(self.handle, ids, len(tokens), pos0, byref(lg), byref(nt)))
        return self._result(lg, nt, want_logits)

    def _result(self, lg, nt, want_logits):
        logits = None
        if want_logits:
            logits = np.empty(self.cfg.vocab, np.float32)
            _check(lib().candy_hip_d2h(self.dev.handle, logits.ctypes.data, lg.value, logits.nbytes))
        return nt.value, logits
