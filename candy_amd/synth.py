"""Seeded synthetic inputs in candy's block formats.

Block layouts follow tensor/internal/cpu/kernels/quantized.go:8-11 (Q4_0), :34-37 (Q8_0),
:55-59 (Q4_K), :70-75 (Q6_K): little-endian, packed, no padding.

The generators draw blocks directly (every byte pattern is a valid block), so the CPU
oracle and the GPU see byte-identical weights; parity is defined on those bytes.
"""
from __future__ import annotations

import numpy as np

Q4_0, Q8_0, Q4_K, Q6_K, Q4_0_GGML = 2, 8, 12, 14, 102
# the reference's other block formats (ggml's type ids; *_GGML = the CUDA kernels' element order)
Q4_1, Q4_1_GGML, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K = 3, 103, 6, 7, 10, 11, 13, 15

BLOCK_DTYPES = {
    Q4_0: np.dtype([("d", "<u2"), ("qs", "u1", 16)]),
    Q4_0_GGML: np.dtype([("d", "<u2"), ("qs", "u1", 16)]),
    Q8_0: np.dtype([("d", "<u2"), ("qs", "i1", 32)]),
    Q4_K: np.dtype([("d", "<u2"), ("dmin", "<u2"), ("scales", "u1", 12), ("qs", "u1", 128)]),
    Q6_K: np.dtype([("ql", "u1", 128), ("qh", "u1", 64), ("scales", "i1", 16), ("d", "<u2")]),
    Q4_1: np.dtype([("d", "<u2"), ("m", "<u2"), ("qs", "u1", 16)]),
    Q4_1_GGML: np.dtype([("d", "<u2"), ("m", "<u2"), ("qs", "u1", 16)]),
    Q5_0: np.dtype([("d", "<u2"), ("qh", "u1", 4), ("qs", "u1", 16)]),
    Q5_1: np.dtype([("d", "<u2"), ("m", "<u2"), ("qh", "u1", 4), ("qs", "u1", 16)]),
    Q2_K: np.dtype([("scales", "u1", 16), ("qs", "u1", 64), ("d", "<u2"), ("dmin", "<u2")]),
    Q3_K: np.dtype([("hmask", "u1", 32), ("qs", "u1", 64), ("scales", "u1", 12), ("d", "<u2")]),
    Q5_K: np.dtype([("d", "<u2"), ("dmin", "<u2"), ("scales", "u1", 12), ("qh", "u1", 32), ("qs", "u1", 128)]),
    Q8_K: np.dtype([("d", "<f4"), ("qs", "i1", 256), ("bsums", "<i2", 16)]),
}
BLOCK_ELEMS = {Q4_0: 32, Q4_0_GGML: 32, Q8_0: 32, Q4_K: 256, Q6_K: 256, Q4_1: 32, Q4_1_GGML: 32, Q5_0: 32, Q5_1: 32,
               Q2_K: 256, Q3_K: 256, Q5_K: 256, Q8_K: 256}
BLOCK_BYTES = {k: v.itemsize for k, v in BLOCK_DTYPES.items()}
FORMAT_NAMES = {Q4_0: "q4_0", Q8_0: "q8_0", Q4_K: "q4_k", Q6_K: "q6_k", Q4_0_GGML: "q4_0_ggml", Q4_1: "q4_1",
                Q4_1_GGML: "q4_1_ggml", Q5_0: "q5_0", Q5_1: "q5_1", Q2_K: "q2_k", Q3_K: "q3_k", Q5_K: "q5_k", Q8_K: "q8_k"}
# formats a weight can be contracted in (Q8_K only dequantizes: the reference has no weight vec-dot for it)
MATMUL_FORMATS = (Q4_0, Q4_0_GGML, Q8_0, Q4_K, Q6_K, Q4_1, Q4_1_GGML, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K)

assert BLOCK_BYTES[Q4_0] == 18 and BLOCK_BYTES[Q8_0] == 34
assert BLOCK_BYTES[Q4_K] == 144 and BLOCK_BYTES[Q6_K] == 210
assert [BLOCK_BYTES[f] for f in (Q4_1, Q5_0, Q5_1, Q2_K, Q3_K, Q5_K, Q8_K)] == [20, 22, 24, 84, 110, 176, 292]


def weight_nbytes(fmt: int, rows: int, cols: int) -> int:
    return rows * (cols // BLOCK_ELEMS[fmt]) * BLOCK_BYTES[fmt]


def _half_scales(rng: np.random.Generator, n: int, scale: float) -> np.ndarray:
    """fp16 bit patterns of |N(0,1)| * scale."""
    return (np.abs(rng.standard_normal(n, dtype=np.float32)) * np.float32(scale)).astype(np.float16).view(np.uint16)


def random_blocks(fmt: int, n_blocks: int, seed: int, scale: float = 0.02) -> np.ndarray:
    """n_blocks random blocks as a flat uint8 array.

    Scales are fp16(|N(0,1)|*scale); quants and sub-scales are uniform over every
    representable value (Q8_0 quants over [-127, 127]).
    """
    rng = np.random.Generator(np.random.Philox(seed))
    dt = BLOCK_DTYPES[fmt]
    raw = rng.integers(0, 256, size=n_blocks * dt.itemsize, dtype=np.uint8)
    blk = raw.view(dt)
    if fmt == Q8_K:
        blk["d"] = np.abs(rng.standard_normal(n_blocks, dtype=np.float32)) * np.float32(scale)
        blk["qs"] = rng.integers(-127, 128, size=(n_blocks, 256), dtype=np.int8)
        blk["bsums"] = blk["qs"].reshape(n_blocks, 16, 16).astype(np.int16).sum(axis=2)
        return raw
    blk["d"] = _half_scales(rng, n_blocks, scale)
    if "dmin" in dt.names:
        blk["dmin"] = _half_scales(rng, n_blocks, scale)
    if "m" in dt.names:  # the minimum of Q4_1 / Q5_1 blocks takes either sign
        m = rng.standard_normal(n_blocks, dtype=np.float32) * np.float32(scale * 4)
        blk["m"] = m.astype(np.float16).view(np.uint16)
    if fmt == Q8_0:
        blk["qs"] = rng.integers(-127, 128, size=(n_blocks, 32), dtype=np.int8)
    return raw


def random_weight(fmt: int, rows: int, cols: int, seed: int, scale: float = 0.02) -> np.ndarray:
    assert cols % BLOCK_ELEMS[fmt] == 0
    return random_blocks(fmt, rows * (cols // BLOCK_ELEMS[fmt]), seed, scale)


def random_activations(m: int, k: int, seed: int) -> np.ndarray:
    rng = np.random.Generator(np.random.Philox(seed))
    return rng.standard_normal((m, k), dtype=np.float32)


def unit_scale(fmt: int, target_std: float = 0.02) -> float:
    """`scale` for random_blocks that makes dequantized weights roughly target_std wide.

    With uniform quants and sub-scales the dequantized magnitude is about
    scale * E|N| * (typical integer magnitude of the format)."""
    typical = {Q4_0: 4.6, Q4_0_GGML: 4.6, Q8_0: 73.0, Q4_K: 300.0, Q6_K: 1400.0, Q4_1: 8.0, Q4_1_GGML: 8.0, Q5_0: 9.2,
               Q5_1: 16.0, Q2_K: 14.0, Q3_K: 40.0, Q5_K: 600.0, Q8_K: 73.0}[fmt]
    return target_std / (0.8 * typical)
