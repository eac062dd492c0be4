"""GGUF files as a source of device-resident quantized weights.

candy has no model file reader for its block formats (the structs of
tensor/internal/cpu/kernels/quantized.go:8-75 are the ggml ones, byte for byte); GGUF is the
container those blocks are published in.  This module reads the container (versions 2 and 3),
hands the tensors out as the raw block bytes the device path consumes unchanged, and builds the
Llama-style decoder from a file.  A small writer produces files of the same layout (synthetic
models, fixtures).

Layout (little-endian): magic "GGUF", u32 version, u64 tensor count, u64 metadata count, the
metadata key/value pairs, the tensor infos (name, dims innermost first, ggml type, offset), zero
padding to `general.alignment` (default 32), then the tensor data, each tensor aligned likewise.

Two conventions differ between a GGUF Llama and candy's kernels, and are bridged here:
  * Q4_0: the file holds ggml's element order (low nibbles are elements 0..15, high nibbles 16..31,
    tensor/internal/cuda/kernels/quantized.cu:862-866); candy's CPU order (quantized.go:87-92)
    interleaves them.  File tensors of type Q4_0 are therefore uploaded as CANDY_HIP_Q4_0_GGML.
  * Rope: converters permute the rows of attn_q / attn_k so that rotating adjacent pairs (2i, 2i+1)
    equals the original model; candy's Rope (reduce.go:3987-4006) rotates pairs (i, i + d/2).
    `unpermute_qk` moves whole rows (blocks are row-contiguous) back to the half-split order.
"""
from __future__ import annotations

import struct
from dataclasses import dataclass

import numpy as np

from . import synth

MAGIC = b"GGUF"
DEFAULT_ALIGNMENT = 32

# ggml tensor types: id -> (elements per block, bytes per block)
GGML_F32, GGML_F16, GGML_Q4_0, GGML_Q8_0, GGML_Q4_K, GGML_Q6_K = 0, 1, 2, 8, 12, 14
GGML_TYPES = {
    0: ("F32", 1, 4), 1: ("F16", 1, 2), 2: ("Q4_0", 32, 18), 3: ("Q4_1", 32, 20), 6: ("Q5_0", 32, 22),
    7: ("Q5_1", 32, 24), 8: ("Q8_0", 32, 34), 9: ("Q8_1", 32, 36), 10: ("Q2_K", 256, 84), 11: ("Q3_K", 256, 110),
    12: ("Q4_K", 256, 144), 13: ("Q5_K", 256, 176), 14: ("Q6_K", 256, 210), 15: ("Q8_K", 256, 292),
}
# file type -> format id of the device path
DEVICE_FORMATS = {GGML_Q4_0: synth.Q4_0_GGML, GGML_Q8_0: synth.Q8_0, GGML_Q4_K: synth.Q4_K, GGML_Q6_K: synth.Q6_K,
                  # files hold Q4_1 in ggml's element order too; the other ids are the device's own
                  3: synth.Q4_1_GGML, 6: synth.Q5_0, 7: synth.Q5_1, 10: synth.Q2_K, 11: synth.Q3_K, 13: synth.Q5_K,
                  15: synth.Q8_K}

# metadata value types
_U8, _I8, _U16, _I16, _U32, _I32, _F32, _BOOL, _STR, _ARR, _U64, _I64, _F64 = range(13)
_SCALARS = {_U8: "<B", _I8: "<b", _U16: "<H", _I16: "<h", _U32: "<I", _I32: "<i", _F32: "<f", _BOOL: "<?",
            _U64: "<Q", _I64: "<q", _F64: "<d"}


class GGUFError(ValueError):
    pass


@dataclass
class TensorInfo:
    name: str
    shape: tuple      # ggml order: shape[0] is the innermost (contiguous) dimension
    ggml_type: int
    offset: int       # relative to the start of the data section
    nbytes: int

    @property
    def cols(self) -> int:
        return int(self.shape[0])

    @property
    def rows(self) -> int:
        return int(np.prod(self.shape[1:], dtype=np.int64)) if len(self.shape) > 1 else 1


class _Reader:
    def __init__(self, buf):
        self.buf, self.pos = buf, 0

    def take(self, fmt: str):
        size = struct.calcsize(fmt)
        if self.pos + size > len(self.buf):
            raise GGUFError("file ends inside the header")
        (v,) = struct.unpack_from(fmt, self.buf, self.pos)
        self.pos += size
        return v

    def string(self) -> str:
        n = self.take("<Q")
        if self.pos + n > len(self.buf):
            raise GGUFError("file ends inside a string")
        s = bytes(self.buf[self.pos:self.pos + n]).decode("utf-8", errors="replace")
        self.pos += n
        return s

    def value(self, vtype: int):
        if vtype in _SCALARS:
            return self.take(_SCALARS[vtype])
        if vtype == _STR:
            return self.string()
        if vtype == _ARR:
            etype, n = self.take("<I"), self.take("<Q")
            if etype in _SCALARS and etype != _BOOL:
                dt = np.dtype(_SCALARS[etype])
                if self.pos + n * dt.itemsize > len(self.buf):
                    raise GGUFError("file ends inside an array")
                arr = np.frombuffer(self.buf, dt, n, self.pos).copy()
                self.pos += n * dt.itemsize
                return arr
            return [self.value(etype) for _ in range(n)]
        raise GGUFError(f"unknown metadata value type {vtype}")


class GGUFFile:
    """A parsed GGUF file; tensor data stays memory-mapped."""

    def __init__(self, path: str):
        self.path = path
        self.data = np.memmap(path, np.uint8, "r")
        r = _Reader(self.data)
        if len(self.data) < 24 or bytes(self.data[:4]) != MAGIC:
            raise GGUFError("not a GGUF file (bad magic)")
        r.pos = 4
        self.version = r.take("<I")
        if self.version not in (2, 3):
            raise GGUFError(f"unsupported GGUF version {self.version}")
        n_tensors, n_kv = r.take("<Q"), r.take("<Q")
        self.metadata = {}
        for _ in range(n_kv):
            key = r.string()
            self.metadata[key] = r.value(r.take("<I"))
        self.alignment = int(self.metadata.get("general.alignment", DEFAULT_ALIGNMENT))
        if self.alignment <= 0 or self.alignment & (self.alignment - 1):
            raise GGUFError(f"alignment {self.alignment} is not a power of two")
        self.tensors = {}
        for _ in range(n_tensors):
            name = r.string()
            n_dims = r.take("<I")
            if n_dims > 4:
                raise GGUFError(f"tensor {name}: {n_dims} dimensions")
            shape = tuple(r.take("<Q") for _ in range(n_dims))
            gtype, offset = r.take("<I"), r.take("<Q")
            if gtype not in GGML_TYPES:
                raise GGUFError(f"tensor {name}: unknown ggml type {gtype}")
            _, elems, bsize = GGML_TYPES[gtype]
            count = int(np.prod(shape, dtype=np.int64)) if shape else 1
            if shape and shape[0] % elems:
                raise GGUFError(f"tensor {name}: row length {shape[0]} is not a multiple of the block size {elems}")
            if offset % self.alignment:
                raise GGUFError(f"tensor {name}: offset {offset} is not aligned to {self.alignment}")
            self.tensors[name] = TensorInfo(name, shape, gtype, offset, count // elems * bsize)
        self.data_start = (r.pos + self.alignment - 1) // self.alignment * self.alignment
        for t in self.tensors.values():
            if self.data_start + t.offset + t.nbytes > len(self.data):
                raise GGUFError(f"tensor {t.name}: data runs past the end of the file")

    def raw(self, name: str) -> np.ndarray:
        """The tensor's bytes exactly as stored (a view into the mapping)."""
        t = self._info(name)
        start = self.data_start + t.offset
        return self.data[start:start + t.nbytes]

    def f32(self, name: str) -> np.ndarray:
        """An F32 or F16 tensor as float32, shaped rows x cols."""
        t = self._info(name)
        if t.ggml_type == GGML_F32:
            a = self.raw(name).view("<f4").astype(np.float32)
        elif t.ggml_type == GGML_F16:
            a = self.raw(name).view("<f2").astype(np.float32)
        else:
            raise GGUFError(f"tensor {name} is {GGML_TYPES[t.ggml_type][0]}, not a float tensor")
        return a.reshape(t.rows, t.cols) if len(t.shape) > 1 else a

    def blocks(self, name: str):
        """(device format id, rows, cols, block bytes) of a quantized matrix, in the file's own layout."""
        t = self._info(name)
        if t.ggml_type not in DEVICE_FORMATS:
            raise GGUFError(f"tensor {name}: type {GGML_TYPES[t.ggml_type][0]} has no device kernels "
                            "(Q4_0, Q4_1, Q5_0, Q5_1, Q8_0, Q2_K ... Q6_K, Q8_K do)")
        return DEVICE_FORMATS[t.ggml_type], t.rows, t.cols, self.raw(name)

    def _info(self, name: str) -> TensorInfo:
        if name not in self.tensors:
            raise GGUFError(f"no tensor named {name}")
        return self.tensors[name]


# ------------------------------------------------------------------ writer

def _pack_string(s: str) -> bytes:
    b = s.encode("utf-8")
    return struct.pack("<Q", len(b)) + b


def _pack_value(v) -> bytes:
    if isinstance(v, bool):
        return struct.pack("<I?", _BOOL, v)
    if isinstance(v, int):
        return struct.pack("<IQ", _U64, v) if v >= 2 ** 32 else struct.pack("<II", _U32, v) if v >= 0 \
            else struct.pack("<Iq", _I64, v)
    if isinstance(v, float):
        return struct.pack("<If", _F32, v)
    if isinstance(v, str):
        return struct.pack("<I", _STR) + _pack_string(v)
    if isinstance(v, np.ndarray):
        codes = {np.dtype("<i4"): _I32, np.dtype("<u4"): _U32, np.dtype("<f4"): _F32, np.dtype("<i8"): _I64}
        if v.dtype not in codes:
            raise GGUFError(f"no GGUF array type for dtype {v.dtype}")
        return struct.pack("<IIQ", _ARR, codes[v.dtype], v.size) + v.tobytes()
    if isinstance(v, (list, tuple)) and all(isinstance(e, str) for e in v):
        return struct.pack("<IIQ", _ARR, _STR, len(v)) + b"".join(_pack_string(e) for e in v)
    raise GGUFError(f"cannot store metadata value of type {type(v).__name__}")


def write_gguf(path: str, metadata: dict, tensors: list, alignment: int = DEFAULT_ALIGNMENT) -> None:
    """tensors: [(name, ggml_type, shape in ggml order, bytes-like)]."""
    meta = dict(metadata)
    if alignment != DEFAULT_ALIGNMENT:
        meta["general.alignment"] = alignment
    head = bytearray(MAGIC + struct.pack("<IQQ", 3, len(tensors), len(meta)))
    for k, v in meta.items():
        head += _pack_string(k) + _pack_value(v)
    offset, placed = 0, []
    for name, gtype, shape, data in tensors:
        data = np.ascontiguousarray(data).view(np.uint8).reshape(-1)
        _, elems, bsize = GGML_TYPES[gtype]
        if shape and shape[0] % elems:
            raise GGUFError(f"tensor {name}: row length {shape[0]} is not a multiple of the block size {elems}")
        want = int(np.prod(shape, dtype=np.int64)) // elems * bsize
        if data.size != want:
            raise GGUFError(f"tensor {name}: {data.size} bytes for shape {tuple(shape)}, expected {want}")
        head += _pack_string(name) + struct.pack("<I", len(shape)) + b"".join(struct.pack("<Q", int(d)) for d in shape)
        head += struct.pack("<IQ", gtype, offset)
        placed.append((offset, data))
        offset = (offset + data.size + alignment - 1) // alignment * alignment
    with open(path, "wb") as f:
        f.write(head)
        f.write(b"\0" * (-len(head) % alignment))
        pos = 0
        for off, data in placed:
            f.write(b"\0" * (off - pos))
            f.write(data.tobytes())
            pos = off + data.size


# ------------------------------------------------------------------ Llama from a file

def unpermute_qk(blocks: np.ndarray, rows: int, n_head: int) -> np.ndarray:
    """Undo the converters' row permutation of attn_q / attn_k.

    File order per head: rows (0, d/2, 1, d/2+1, ...) of the original; returns the original order
    (first half, then second half), which is what a Rope over pairs (i, i + d/2) expects.
    """
    if rows % (2 * n_head):
        raise GGUFError(f"{rows} rows do not split into {n_head} heads of even size")
    per_row = blocks.size // rows
    b = np.asarray(blocks).reshape(n_head, rows // n_head // 2, 2, per_row)
    return np.ascontiguousarray(b.swapaxes(1, 2)).reshape(-1)


def permute_qk(blocks: np.ndarray, rows: int, n_head: int) -> np.ndarray:
    """The converters' permutation (inverse of `unpermute_qk`)."""
    per_row = blocks.size // rows
    b = np.asarray(blocks).reshape(n_head, 2, rows // n_head // 2, per_row)
    return np.ascontiguousarray(b.swapaxes(1, 2)).reshape(-1)


def llama_config(g: GGUFFile, max_pos: int | None = None) -> dict:
    arch = g.metadata.get("general.architecture", "llama")
    md = g.metadata

    def need(key):
        full = f"{arch}.{key}"
        if full not in md:
            raise GGUFError(f"metadata key {full} is missing")
        return md[full]

    d_model, n_heads = int(need("embedding_length")), int(need("attention.head_count"))
    n_kv = int(md.get(f"{arch}.attention.head_count_kv", n_heads))
    head_dim = int(md.get(f"{arch}.rope.dimension_count", d_model // n_heads))
    embd = g.tensors.get("token_embd.weight")
    if embd is None:
        raise GGUFError("no tensor named token_embd.weight")
    ctx = int(md.get(f"{arch}.context_length", 2048))
    return dict(n_layers=int(need("block_count")), d_model=d_model, n_heads=n_heads, n_kv_heads=n_kv, head_dim=head_dim,
                d_ffn=int(need("feed_forward_length")), vocab=int(md.get(f"{arch}.vocab_size", embd.rows)),
                max_pos=int(max_pos if max_pos is not None else ctx),
                rms_eps=float(md.get(f"{arch}.attention.layer_norm_rms_epsilon", 1e-5)),
                rope_base=float(md.get(f"{arch}.rope.freq_base", 10000.0)))


_LAYER_TENSORS = (("attn_q", "W_Q"), ("attn_k", "W_K"), ("attn_v", "W_V"), ("attn_output", "W_O"),
                  ("ffn_gate", "W_GATE"), ("ffn_up", "W_UP"), ("ffn_down", "W_DOWN"))


def llama_weights(g: GGUFFile, cfg: dict, qk_permuted: bool = True) -> dict:
    """{(kind, layer): (fmt, block bytes) | f32 array} in the order the kernels expect (kinds as in candy_hip.h)."""
    out = {}
    for l in range(cfg["n_layers"]):
        for tname, kind in _LAYER_TENSORS:
            fmt, rows, cols, blk = g.blocks(f"blk.{l}.{tname}.weight")
            if qk_permuted and tname in ("attn_q", "attn_k"):
                blk = unpermute_qk(blk, rows, cfg["n_heads"] if tname == "attn_q" else cfg["n_kv_heads"])
            out[(kind[2:].lower(), l)] = (fmt, np.ascontiguousarray(blk))
        out[("attn_norm", l)] = g.f32(f"blk.{l}.attn_norm.weight").reshape(-1)
        out[("ffn_norm", l)] = g.f32(f"blk.{l}.ffn_norm.weight").reshape(-1)
    out[("out_norm", -1)] = g.f32("output_norm.weight").reshape(-1)
    fmt, _, _, blk = g.blocks("token_embd.weight")
    out[("embed", -1)] = (fmt, np.ascontiguousarray(blk))
    head = "output.weight" if "output.weight" in g.tensors else "token_embd.weight"  # tied embeddings
    fmt, _, _, blk = g.blocks(head)
    out[("head", -1)] = (fmt, np.ascontiguousarray(blk))
    return out


def load_llama(dev, path: str, max_pos: int | None = None, qk_permuted: bool = True):
    """Builds the device decoder from a GGUF file. Returns (model, config, weights as uploaded)."""
    from . import hip

    g = GGUFFile(path)
    cfg = llama_config(g, max_pos)
    weights = llama_weights(g, cfg, qk_permuted)
    qd, kvd = cfg["n_heads"] * cfg["head_dim"], cfg["n_kv_heads"] * cfg["head_dim"]
    shapes = {"q": (qd, cfg["d_model"]), "k": (kvd, cfg["d_model"]), "v": (kvd, cfg["d_model"]),
              "o": (cfg["d_model"], qd), "gate": (cfg["d_ffn"], cfg["d_model"]), "up": (cfg["d_ffn"], cfg["d_model"]),
              "down": (cfg["d_model"], cfg["d_ffn"]), "head": (cfg["vocab"], cfg["d_model"]),
              "embed": (cfg["vocab"], cfg["d_model"])}
    codes = {"q": hip.W_Q, "k": hip.W_K, "v": hip.W_V, "o": hip.W_O, "gate": hip.W_GATE, "up": hip.W_UP,
             "down": hip.W_DOWN, "head": hip.W_HEAD, "embed": hip.W_EMBED, "attn_norm": hip.W_ATTN_NORM,
             "ffn_norm": hip.W_FFN_NORM, "out_norm": hip.W_OUT_NORM}
    model = hip.Llama(dev, **cfg)
    for (kind, layer), w in weights.items():
        if isinstance(w, tuple):
            fmt, blk = w
            rows, cols = shapes[kind]
            want = synth.weight_nbytes(fmt, rows, cols)
            if blk.size != want:
                raise GGUFError(f"{kind} of layer {layer}: {blk.size} bytes, the configuration implies {want}")
            model.set_qweight(codes[kind], layer, dev.qtensor(fmt, rows, cols, blk))
        else:
            model.set_norm(codes[kind], layer, w)
    return model, cfg, weights
