"""A Llama written to a GGUF file the way converters lay it out (ggml-order Q4_0, permuted attn_q / attn_k
rows) and loaded back through candy_amd.gguf decodes like the CPU composition on the original weights."""
import numpy as np
import pytest

from candy_amd import gguf, hip, synth
from oracle import llama_ref
from test_gguf import OTHER_FORMATS, tiny_model

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))


# files hold the 4-bit formats in ggml's element order: the device (and the oracle) read them as the *_GGML ids
FILE_ORDER = {synth.Q4_0: synth.Q4_0_GGML, synth.Q4_1: synth.Q4_1_GGML}


@pytest.mark.parametrize("tied,fmts", [(False, None), (True, None), (False, OTHER_FORMATS)],
                         ids=["untied", "tied", "other-formats"])
def test_model_from_file_matches_cpu_composition(dev, tmp_path, tied, fmts):
    cfg, meta, tensors, orig = tiny_model(seed=7, tied=tied, fmts=fmts)
    path = str(tmp_path / "tiny.gguf")
    gguf.write_gguf(path, meta, tensors)
    model, got_cfg, _ = gguf.load_llama(dev, path)
    assert got_cfg["n_layers"] == 2 and got_cfg["head_dim"] == 64 and got_cfg["vocab"] == cfg["vocab"]
    # the oracle's model is built from the ORIGINAL tensors (half-split q / k rows), not from what the reader returned
    names = {"q": "attn_q", "k": "attn_k", "v": "attn_v", "o": "attn_output", "gate": "ffn_gate", "up": "ffn_up",
             "down": "ffn_down"}
    host = {}
    for l in range(cfg["n_layers"]):
        for kind, tname in names.items():
            fmt, r, c, blk = orig[(tname, l)]
            host[(kind, l)] = (FILE_ORDER.get(fmt, fmt), blk)
        host[("attn_norm", l)], host[("ffn_norm", l)] = orig[("attn_norm", l)], orig[("ffn_norm", l)]
    host[("out_norm", -1)] = orig[("out_norm", -1)]
    host[("embed", -1)] = (orig[("embed", -1)][0], orig[("embed", -1)][3])
    hd = orig[("embed", -1)] if tied else orig[("head", -1)]
    host[("head", -1)] = (hd[0], hd[3])
    ref = llama_ref.LlamaRef({**cfg, "rms_eps": got_cfg["rms_eps"], "rope_base": got_cfg["rope_base"]}, host)
    tokens = [int(t) for t in np.random.default_rng(8).integers(0, cfg["vocab"], 9)]
    for pos, tok in enumerate(tokens):
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
    # Formats whose levels are symmetric about zero (Q5_0, Q3_K ...) leave no common mode in the rows to mask the
    # occasional Q8_0 rounding flip that another f32 summation order causes; over two layers those grow to a few 1e-3
    # (each op alone matches to 1e-6: tests/test_gpu_formats_more.py).  A layout mistake would be of order 1.
    bar = 1e-3 if fmts is None else 5e-3
    nt, logits = model.prefill(tokens, 0)
    assert rel(logits, rlogits) <= bar
    assert nt == int(np.argmax(logits))
    tok = nt
    for pos in range(len(tokens), len(tokens) + 3):
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
        gt, glogits = model.decode(tok, pos)
        assert rel(glogits, rlogits) <= bar
        tok = rt
    # reading the same file without undoing the row permutation gives a different model (the bridge matters)
    wrong, _, _ = gguf.load_llama(dev, path, qk_permuted=False)
    _, wl = wrong.prefill(tokens, 0)
    assert rel(wl, logits.astype(np.float64)) > 1e-2
