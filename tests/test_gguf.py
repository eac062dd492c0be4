"""GGUF container: writer/reader round trips, header validation, the two convention bridges
(Q4_0 element order, attn_q / attn_k row permutation). CPU only."""
import struct

import numpy as np
import pytest

from candy_amd import gguf, synth
from oracle import oracle as o


OTHER_FORMATS = {"attn_q": synth.Q5_K, "attn_k": synth.Q5_0, "attn_v": synth.Q5_1, "attn_output": synth.Q4_1,
                 "ffn_gate": synth.Q3_K, "ffn_up": synth.Q2_K, "ffn_down": synth.Q5_K}


def tiny_model(seed=1, tied=False, fmts=None):
    cfg = dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, head_dim=64, d_ffn=512, vocab=96, max_pos=32,
               rms_eps=1e-6, rope_base=50000.0)
    qd, kvd = 256, 128
    shapes = {"attn_q": (qd, 256), "attn_k": (kvd, 256), "attn_v": (kvd, 256), "attn_output": (256, qd),
              "ffn_gate": (512, 256), "ffn_up": (512, 256), "ffn_down": (256, 512)}
    fmts = fmts or {"attn_q": synth.Q4_K, "attn_k": synth.Q8_0, "attn_v": synth.Q6_K, "attn_output": synth.Q4_K,
                    "ffn_gate": synth.Q4_0, "ffn_up": synth.Q4_K, "ffn_down": synth.Q6_K}
    rng = np.random.default_rng(seed)
    orig, tensors, s = {}, [], seed * 100
    for l in range(cfg["n_layers"]):
        for name, (r, c) in shapes.items():
            blk = synth.random_weight(fmts[name], r, c, seed=(s := s + 1), scale=synth.unit_scale(fmts[name]))
            orig[(name, l)] = (fmts[name], r, c, blk)
            stored = blk
            if name in ("attn_q", "attn_k"):
                stored = gguf.permute_qk(blk, r, cfg["n_heads"] if name == "attn_q" else cfg["n_kv_heads"])
            tensors.append((f"blk.{l}.{name}.weight", fmts[name], (c, r), stored))
        for name in ("attn_norm", "ffn_norm"):
            a = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
            orig[(name, l)] = a
            tensors.append((f"blk.{l}.{name}.weight", gguf.GGML_F32, (256,), a))
    a = (1 + 0.1 * rng.standard_normal(256)).astype(np.float32)
    orig[("out_norm", -1)] = a
    tensors.append(("output_norm.weight", gguf.GGML_F32, (256,), a))
    embd = synth.random_weight(synth.Q8_0, cfg["vocab"], 256, seed=(s := s + 1), scale=synth.unit_scale(synth.Q8_0))
    orig[("embed", -1)] = (synth.Q8_0, cfg["vocab"], 256, embd)
    tensors.append(("token_embd.weight", synth.Q8_0, (256, cfg["vocab"]), embd))
    if not tied:
        head = synth.random_weight(synth.Q6_K, cfg["vocab"], 256, seed=(s := s + 1), scale=synth.unit_scale(synth.Q6_K))
        orig[("head", -1)] = (synth.Q6_K, cfg["vocab"], 256, head)
        tensors.append(("output.weight", synth.Q6_K, (256, cfg["vocab"]), head))
    meta = {"general.architecture": "llama", "general.name": "tiny", "llama.block_count": cfg["n_layers"],
            "llama.embedding_length": 256, "llama.attention.head_count": 4, "llama.attention.head_count_kv": 2,
            "llama.feed_forward_length": 512, "llama.context_length": 32, "llama.rope.dimension_count": 64,
            "llama.attention.layer_norm_rms_epsilon": 1e-6, "llama.rope.freq_base": 50000.0,
            "tokenizer.ggml.tokens": [f"t{i}" for i in range(cfg["vocab"])],
            "tokenizer.ggml.token_type": np.ones(cfg["vocab"], "<i4")}
    return cfg, meta, tensors, orig


@pytest.mark.parametrize("version", [2, 3])
def test_reader_on_bytes_assembled_by_hand_from_the_published_layout(tmp_path, version):
    # Every other test here reads files that write_gguf wrote: a misreading of the format shared by reader and writer
    # would pass them all.  This file is put together byte by byte from the constants of the published GGUF
    # specification (ggml docs/gguf.md), with struct.pack and literal numbers only - nothing from candy_amd.gguf:
    #   header   magic "GGUF" = 0x46554747 little endian, u32 version, u64 tensor count, u64 metadata count
    #   string   u64 length + UTF-8 bytes, no terminator
    #   value    u32 type, then the value; types UINT8 0, INT8 1, UINT16 2, INT16 3, UINT32 4, INT32 5, FLOAT32 6,
    #            BOOL 7 (one byte), STRING 8, ARRAY 9 (u32 element type, u64 count, elements), UINT64 10, INT64 11,
    #            FLOAT64 12
    #   tensor   name string, u32 n_dims, u64 dims[n_dims] (dims[0] the contiguous one), u32 ggml type (F32 0, F16 1,
    #            Q4_0 2, Q8_0 8, Q4_K 12, Q6_K 14, ...), u64 offset from the start of the data section
    #   data     starts at the next multiple of general.alignment (default 32) after the last tensor info; every
    #            tensor offset is a multiple of it
    def gstr(t):
        b = t.encode("utf-8")
        return struct.pack("<Q", len(b)) + b

    kv = [
        gstr("general.architecture") + struct.pack("<I", 8) + gstr("llama"),
        gstr("general.alignment") + struct.pack("<II", 4, 64),
        gstr("t.u8") + struct.pack("<IB", 0, 200),
        gstr("t.i8") + struct.pack("<Ib", 1, -100),
        gstr("t.u16") + struct.pack("<IH", 2, 60000),
        gstr("t.i16") + struct.pack("<Ih", 3, -30000),
        gstr("t.i32") + struct.pack("<Ii", 5, -2000000000),
        gstr("t.f32") + struct.pack("<If", 6, 0.15625),
        gstr("t.bool") + struct.pack("<IB", 7, 1),
        gstr("t.u64") + struct.pack("<IQ", 10, 2 ** 63 + 5),
        gstr("t.i64") + struct.pack("<Iq", 11, -(2 ** 62)),
        gstr("t.f64") + struct.pack("<Id", 12, 1.0 / 3.0),
        gstr("t.strs") + struct.pack("<IIQ", 9, 8, 3) + gstr("a") + gstr("") + gstr("h\u00e9llo"),
        gstr("t.ints") + struct.pack("<IIQ", 9, 5, 4) + struct.pack("<4i", 7, -8, 9, -10),
        gstr("t.floats") + struct.pack("<IIQ", 9, 6, 2) + struct.pack("<2f", 0.5, -2.0),
    ]
    # tensor 0: F32 vector of 8 values (32 bytes) at offset 0; tensor 1: Q8_0 matrix, 64 columns x 2 rows = 4 blocks of
    # 34 bytes, at the next multiple of 64; tensor 2: Q4_K 256 columns x 1 row = 144 bytes, after 136 -> offset 256
    vec = struct.pack("<8f", *[0.25 * i for i in range(8)])
    q8 = bytes((37 * i + 11) % 256 for i in range(4 * 34))
    q4k = bytes((91 * i + 3) % 256 for i in range(144))
    infos = [
        gstr("vec.weight") + struct.pack("<I", 1) + struct.pack("<Q", 8) + struct.pack("<IQ", 0, 0),
        gstr("blk.0.q8.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 64, 2) + struct.pack("<IQ", 8, 64),
        gstr("blk.0.q4k.weight") + struct.pack("<I", 2) + struct.pack("<QQ", 256, 1) + struct.pack("<IQ", 12, 256),
    ]
    head = b"GGUF" + struct.pack("<IQQ", version, len(infos), len(kv)) + b"".join(kv) + b"".join(infos)
    assert head[:4] == struct.pack("<I", 0x46554747)
    pad = (-len(head)) % 64
    data = vec + b"\x00" * 32 + q8 + b"\x00" * (256 - 64 - len(q8)) + q4k
    path = tmp_path / "hand.gguf"
    path.write_bytes(head + b"\x00" * pad + data)

    g = gguf.GGUFFile(str(path))
    assert g.version == version and g.alignment == 64 and g.data_start == len(head) + pad
    m = g.metadata
    assert m["general.architecture"] == "llama"
    assert (m["t.u8"], m["t.i8"], m["t.u16"], m["t.i16"], m["t.i32"]) == (200, -100, 60000, -30000, -2000000000)
    assert m["t.f32"] == 0.15625 and m["t.bool"] is True and m["t.f64"] == 1.0 / 3.0
    assert m["t.u64"] == 2 ** 63 + 5 and m["t.i64"] == -(2 ** 62)
    assert list(m["t.strs"]) == ["a", "", "h\u00e9llo"]
    assert list(m["t.ints"]) == [7, -8, 9, -10] and list(m["t.floats"]) == [0.5, -2.0]
    assert set(g.tensors) == {"vec.weight", "blk.0.q8.weight", "blk.0.q4k.weight"}
    t = g.tensors["blk.0.q8.weight"]
    assert (t.shape, t.ggml_type, t.offset, t.nbytes, t.rows, t.cols) == ((64, 2), 8, 64, 136, 2, 64)
    assert bytes(g.raw("blk.0.q8.weight")) == q8 and bytes(g.raw("blk.0.q4k.weight")) == q4k
    assert np.array_equal(g.f32("vec.weight"), np.arange(8, dtype=np.float32) * 0.25)
    fmt, rows, cols, blocks = g.blocks("blk.0.q8.weight")
    assert (fmt, rows, cols) == (synth.Q8_0, 2, 64)
    # the block bytes mean what the format says: fp16 scale first, then 32 int8 quants (quantized.go:34-37)
    d = np.frombuffer(q8[:2], "<f2")[0].astype(np.float32)
    want = d * np.frombuffer(q8[2:34], np.int8).astype(np.float32)
    assert np.array_equal(o.dequantize(fmt, np.frombuffer(bytes(blocks), np.uint8))[:32], want)
    fmt, rows, cols, blocks = g.blocks("blk.0.q4k.weight")
    assert (fmt, rows, cols, len(blocks)) == (synth.Q4_K, 1, 256, 144)


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_round_trip_keeps_every_byte(tmp_path, alignment):
    cfg, meta, tensors, _ = tiny_model()
    path = str(tmp_path / "m.gguf")
    gguf.write_gguf(path, meta, tensors, alignment=alignment)
    g = gguf.GGUFFile(path)
    assert g.version == 3 and g.alignment == alignment and g.data_start % alignment == 0
    assert g.metadata["general.name"] == "tiny" and g.metadata["llama.block_count"] == 2
    assert abs(g.metadata["llama.rope.freq_base"] - 50000.0) < 1e-3
    assert g.metadata["tokenizer.ggml.tokens"][5] == "t5" and len(g.metadata["tokenizer.ggml.tokens"]) == cfg["vocab"]
    assert np.array_equal(g.metadata["tokenizer.ggml.token_type"], np.ones(cfg["vocab"], np.int32))
    assert set(g.tensors) == {t[0] for t in tensors}
    for name, gtype, shape, data in tensors:
        t = g.tensors[name]
        assert t.shape == tuple(shape) and t.ggml_type == gtype and t.offset % alignment == 0
        assert np.array_equal(g.raw(name), np.ascontiguousarray(data).view(np.uint8).reshape(-1))
    t = g.tensors["blk.1.ffn_down.weight"]
    assert (t.rows, t.cols) == (256, 512) and t.nbytes == synth.weight_nbytes(synth.Q6_K, 256, 512)


def test_llama_weights_come_back_in_kernel_order(tmp_path):
    cfg, meta, tensors, orig = tiny_model(seed=2)
    path = str(tmp_path / "m.gguf")
    gguf.write_gguf(path, meta, tensors)
    g = gguf.GGUFFile(path)
    got_cfg = gguf.llama_config(g)
    assert got_cfg == {**cfg, "rms_eps": pytest.approx(1e-6), "rope_base": pytest.approx(50000.0)}
    assert gguf.llama_config(g, max_pos=8)["max_pos"] == 8
    w = gguf.llama_weights(g, got_cfg)
    names = {"q": "attn_q", "k": "attn_k", "v": "attn_v", "o": "attn_output", "gate": "ffn_gate", "up": "ffn_up",
             "down": "ffn_down"}
    for l in range(cfg["n_layers"]):
        for kind, tname in names.items():
            fmt, r, c, blk = orig[(tname, l)]
            gfmt, gblk = w[(kind, l)]
            # Q4_0 in a file is ggml's element order: a format id of its own on the device
            assert gfmt == (synth.Q4_0_GGML if fmt == synth.Q4_0 else fmt)
            assert np.array_equal(gblk, blk), (kind, l)  # q / k rows are back in half-split order
        assert np.array_equal(w[("attn_norm", l)], orig[("attn_norm", l)])
    assert np.array_equal(w[("head", -1)][1], orig[("head", -1)][3]) and w[("head", -1)][0] == synth.Q6_K
    assert np.array_equal(w[("embed", -1)][1], orig[("embed", -1)][3])
    # without the un-permutation the file's own row order comes back
    raw = gguf.llama_weights(g, got_cfg, qk_permuted=False)
    assert not np.array_equal(raw[("q", 0)][1], orig[("attn_q", 0)][3])
    assert np.array_equal(raw[("v", 0)][1], orig[("attn_v", 0)][3])


def test_tied_embeddings_serve_as_head(tmp_path):
    cfg, meta, tensors, orig = tiny_model(seed=3, tied=True)
    path = str(tmp_path / "m.gguf")
    gguf.write_gguf(path, meta, tensors)
    g = gguf.GGUFFile(path)
    w = gguf.llama_weights(g, gguf.llama_config(g))
    assert w[("head", -1)][0] == synth.Q8_0 and np.array_equal(w[("head", -1)][1], orig[("embed", -1)][3])


def test_qk_permutation_is_the_converters_row_map():
    n_head, hd, per_row = 3, 8, 5
    rows = n_head * hd
    blk = np.arange(rows * per_row, dtype=np.uint8).reshape(rows, per_row)
    perm = gguf.permute_qk(blk.reshape(-1), rows, n_head).reshape(rows, per_row)
    for h in range(n_head):
        for i in range(hd // 2):
            # file row 2i is the original row i, file row 2i+1 the original row i + d/2
            assert np.array_equal(perm[h * hd + 2 * i], blk[h * hd + i])
            assert np.array_equal(perm[h * hd + 2 * i + 1], blk[h * hd + hd // 2 + i])
    assert np.array_equal(gguf.unpermute_qk(perm.reshape(-1), rows, n_head).reshape(rows, per_row), blk)
    with pytest.raises(gguf.GGUFError, match="heads"):
        gguf.unpermute_qk(blk.reshape(-1), rows, 5)


def test_file_q4_0_is_ggml_element_order(tmp_path):
    # a Q4_0 block whose low nibbles are 0..15 and high nibbles 15..0, d = 1: ggml order puts the 16 low
    # nibbles first (quantized.cu:862-866), candy's CPU order interleaves (quantized.go:87-92)
    blk = np.zeros(1, synth.BLOCK_DTYPES[synth.Q4_0])
    blk["d"] = np.float16(1.0).view(np.uint16)
    blk["qs"] = (np.arange(16) | ((15 - np.arange(16)) << 4)).astype(np.uint8)
    path = str(tmp_path / "q.gguf")
    gguf.write_gguf(path, {}, [("w", gguf.GGML_Q4_0, (32, 1), blk)])
    fmt, rows, cols, raw = gguf.GGUFFile(path).blocks("w")
    assert (fmt, rows, cols) == (synth.Q4_0_GGML, 1, 32)
    y = o.dequantize(fmt, np.array(raw))
    assert np.array_equal(y[:16], np.arange(16) - 8.0) and np.array_equal(y[16:], (15 - np.arange(16)) - 8.0)
    y_cpu = o.dequantize(synth.Q4_0, np.array(raw))
    assert np.array_equal(y_cpu[0::2], np.arange(16) - 8.0)


def test_f16_and_f32_tensors(tmp_path):
    a = np.linspace(-2, 2, 64, dtype=np.float32)
    path = str(tmp_path / "f.gguf")
    gguf.write_gguf(path, {"x": 7, "neg": -3, "big": 2 ** 40, "flag": True, "pi": 3.25},
                    [("a32", gguf.GGML_F32, (16, 4), a), ("a16", gguf.GGML_F16, (64,), a.astype(np.float16))])
    g = gguf.GGUFFile(path)
    assert g.metadata == {"x": 7, "neg": -3, "big": 2 ** 40, "flag": True, "pi": 3.25}
    assert g.f32("a32").shape == (4, 16) and np.array_equal(g.f32("a32").reshape(-1), a)
    assert np.array_equal(g.f32("a16"), a.astype(np.float16).astype(np.float32))
    with pytest.raises(gguf.GGUFError, match="no device kernels|F32"):
        g.blocks("a32")


def test_header_validation(tmp_path):
    cfg, meta, tensors, _ = tiny_model()
    good = str(tmp_path / "g.gguf")
    gguf.write_gguf(good, meta, tensors)
    data = bytearray(open(good, "rb").read())

    def variant(name, edit):
        b = bytearray(data)
        edit(b)
        p = str(tmp_path / name)
        open(p, "wb").write(b)
        return p

    with pytest.raises(gguf.GGUFError, match="magic"):
        gguf.GGUFFile(variant("magic", lambda b: b.__setitem__(slice(0, 4), b"GGML")))
    with pytest.raises(gguf.GGUFError, match="version"):
        gguf.GGUFFile(variant("ver", lambda b: b.__setitem__(slice(4, 8), struct.pack("<I", 1))))
    with pytest.raises(gguf.GGUFError, match="past the end|ends inside"):
        gguf.GGUFFile(variant("trunc", lambda b: b.__delitem__(slice(len(b) - 1000, len(b)))))
    with pytest.raises(gguf.GGUFError, match="ends inside"):
        gguf.GGUFFile(variant("short", lambda b: b.__delitem__(slice(200, len(b)))))
    # a tensor of a ggml type that exists but has no kernels here (Q8_1 = 9); Q5_K = 13 has
    p = str(tmp_path / "q81.gguf")
    gguf.write_gguf(p, {}, [("w", 9, (32, 2), np.zeros(2 * 36, np.uint8)), ("v", 13, (256, 2), np.zeros(2 * 176, np.uint8))])
    g = gguf.GGUFFile(p)
    assert g.tensors["w"].nbytes == 72 and g.tensors["v"].nbytes == 352
    with pytest.raises(gguf.GGUFError, match="no device kernels"):
        g.blocks("w")
    assert g.blocks("v")[:3] == (synth.Q5_K, 2, 256)
    with pytest.raises(gguf.GGUFError, match="no tensor named"):
        g.raw("missing")
    with pytest.raises(gguf.GGUFError, match="multiple of the block size"):
        gguf.write_gguf(str(tmp_path / "bad.gguf"), {}, [("w", gguf.GGML_Q4_K, (100, 1), np.zeros(144, np.uint8))])
        gguf.GGUFFile(str(tmp_path / "bad.gguf"))
    with pytest.raises(gguf.GGUFError, match="is missing"):
        p2 = str(tmp_path / "nometa.gguf")
        gguf.write_gguf(p2, {"general.architecture": "llama"}, tensors)
        gguf.llama_config(gguf.GGUFFile(p2))
