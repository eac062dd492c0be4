"""Decode-step parity: the device decoder against the CPU composition of oracle ops on a
reduced-depth Llama with full-width layers, plus properties at the full 7B shape."""
import numpy as np
import pytest

from candy_amd import hip, synth
from oracle import llama_ref

pytestmark = pytest.mark.gpu

KINDS = {"q": hip.W_Q, "k": hip.W_K, "v": hip.W_V, "o": hip.W_O, "gate": hip.W_GATE, "up": hip.W_UP,
         "down": hip.W_DOWN, "head": hip.W_HEAD, "embed": hip.W_EMBED,
         "attn_norm": hip.W_ATTN_NORM, "ffn_norm": hip.W_FFN_NORM, "out_norm": hip.W_OUT_NORM}


@pytest.fixture(scope="module")
def dev():
    d = hip.Device(0)
    yield d
    d.close()


def quantized_normal(fmt, rows, cols, seed):
    from oracle import oracle
    x = np.random.default_rng(seed).standard_normal((rows, cols)).astype(np.float32) * np.float32(0.02)
    return oracle.quantize(fmt, x)


def build(dev, cfg, fmts, seed=0, from_normal=False):
    """Random-init weights in the given formats, on the host (for the oracle) and the device.
    from_normal: the weights are drawn from N(0, 0.02) and quantized (by the oracle's quantizer) instead of
    being random blocks."""
    c = cfg
    qd, kvd = c["n_heads"] * c["head_dim"], c["n_kv_heads"] * c["head_dim"]
    shapes = {"q": (qd, c["d_model"]), "k": (kvd, c["d_model"]), "v": (kvd, c["d_model"]), "o": (c["d_model"], qd),
              "gate": (c["d_ffn"], c["d_model"]), "up": (c["d_ffn"], c["d_model"]), "down": (c["d_model"], c["d_ffn"])}
    rng = np.random.default_rng(seed)
    host, model = {}, hip.Llama(dev, **c)
    s = seed * 1000
    for l in range(c["n_layers"]):
        for kind, (r, k) in shapes.items():
            fmt = fmts.get(kind, fmts["default"])
            if from_normal:
                blocks = quantized_normal(fmt, r, k, seed=(s := s + 1))
            else:
                blocks = synth.random_weight(fmt, r, k, seed=(s := s + 1), scale=synth.unit_scale(fmt))
            host[(kind, l)] = (fmt, blocks)
            model.set_qweight(KINDS[kind], l, dev.qtensor(fmt, r, k, blocks))
        for kind in ("attn_norm", "ffn_norm"):
            a = (1 + 0.1 * rng.standard_normal(c["d_model"])).astype(np.float32)
            host[(kind, l)] = a
            model.set_norm(KINDS[kind], l, a)
    a = (1 + 0.1 * rng.standard_normal(c["d_model"])).astype(np.float32)
    host[("out_norm", -1)] = a
    model.set_norm(hip.W_OUT_NORM, -1, a)
    for kind in ("head", "embed"):
        fmt = fmts.get(kind, fmts["default"])
        if from_normal:
            blocks = quantized_normal(fmt, c["vocab"], c["d_model"], seed=(s := s + 1))
        else:
            blocks = synth.random_weight(fmt, c["vocab"], c["d_model"], seed=(s := s + 1), scale=synth.unit_scale(fmt))
        host[(kind, -1)] = (fmt, blocks)
        model.set_qweight(KINDS[kind], -1, dev.qtensor(fmt, c["vocab"], c["d_model"], blocks))
    return host, model


def rel(got, want):
    return float(np.max(np.abs(got.astype(np.float64) - want)) / np.max(np.abs(want)))


@pytest.mark.parametrize("name,cfg,fmts", [
    ("7b-shaped", dict(n_layers=2, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=11008, vocab=2048,
                       max_pos=48, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}),
    ("8b-shaped-gqa", dict(n_layers=2, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ffn=14336, vocab=2048,
                           max_pos=48, rms_eps=1e-5, rope_base=500000.0),
     {"default": synth.Q4_K, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}),
    ("small-mixed", dict(n_layers=3, d_model=512, n_heads=8, n_kv_heads=2, head_dim=64, d_ffn=1024, vocab=512,
                         max_pos=16, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q8_0, "gate": synth.Q4_0, "down": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q4_K}),
    # Q5_K_M-like: Q5_K linears on the fused kernels' lighter shapes (one row, or row pair, per wavefront)
    ("q5_k-q6k-down", dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=4, head_dim=64, d_ffn=1536, vocab=512,
                           max_pos=16, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q5_K, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}),
    # the formats without fused decode kernels: every Linear falls back to quantize + general matvec (+ add)
    ("other-formats", dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=4, head_dim=64, d_ffn=1024, vocab=512,
                           max_pos=16, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q5_K, "q": synth.Q5_0, "k": synth.Q4_1, "v": synth.Q5_1, "gate": synth.Q3_K, "up": synth.Q2_K,
      "head": synth.Q4_1_GGML, "embed": synth.Q8_K}),
])
def test_decode_steps_match_cpu_composition(dev, name, cfg, fmts):
    host, model = build(dev, cfg, fmts, seed=3)
    ref = llama_ref.LlamaRef(cfg, host)
    rng = np.random.default_rng(5)
    tokens = rng.integers(0, cfg["vocab"], 4)
    for pos, tok in enumerate(tokens):
        nt, logits = model.decode(int(tok), pos)
        rt, rlogits, _ = ref.step(ref.embed(int(tok)), pos)
        # logits within 1e-3 of the CPU result (max-norm); the Q8_0 re-quantization of every
        # activation amplifies f32 rounding differences a little, layer after layer
        assert rel(logits, rlogits) <= 1e-3, (name, pos)
        top2 = np.sort(rlogits)[-2:]
        if top2[1] - top2[0] > 2e-3 * np.max(np.abs(rlogits)):
            assert nt == rt, (name, pos)
        assert nt == int(np.argmax(logits))
    # the device KV cache holds what the CPU composition wrote
    kptr, vptr, nbytes = model.kv_cache()
    kc = np.empty(nbytes // 4, np.float32)
    hip._check(hip.lib().candy_hip_d2h(dev.handle, kc.ctypes.data, kptr, nbytes))
    kc = kc.reshape(ref.k_cache.shape)
    assert rel(kc[:, :, :len(tokens)], ref.k_cache[:, :, :len(tokens)].astype(np.float64)) <= 1e-3


def test_decode_with_weights_quantized_from_normal(dev):
    # The benchmark's model in small: every matrix drawn from N(0, 0.02) and then quantized (Q4_K linears, Q6_K
    # head, Q8_0 embedding), full-width layers.
    # Each op of the step matches the CPU to about 3e-7 on the same input, but the step as a whole is not a
    # continuous function of its input: every Linear re-quantizes its activations to Q8_0, an f32 difference in
    # the last place flips a rounding here and there, and a flipped level (1/127 of a block's range) is a far
    # larger difference for the next quantizer, which flips more: the difference between two correct
    # implementations grows about twentyfold per Linear until it reaches the size of the quantizer's own noise and
    # stays there.  With such weights that is reached within two layers (with the random-block weights of the other
    # tests, whose rows have a large common mode, it is not).  So the bar here is that noise itself: the device and
    # the CPU composition must differ by less than the CPU composition differs from the same model run WITHOUT the
    # activation quantizer (dequantized weights, f32 activations), and the first layer's k/v, which only one
    # quantizer precedes, must agree to 1e-3.
    cfg = dict(n_layers=2, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=11008, vocab=1024,
               max_pos=16, rms_eps=1e-5, rope_base=10000.0)
    fm = {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    host, model = build(dev, cfg, fm, seed=40, from_normal=True)
    w = np.random.default_rng(41 * 1000 + 1).standard_normal((4096, 4096)).astype(np.float32) * np.float32(0.02)
    assert np.array_equal(dev.quantize(synth.Q4_K, w), quantized_normal(synth.Q4_K, 4096, 4096, 41 * 1000 + 1))
    ref = llama_ref.LlamaRef(cfg, host)
    plain = llama_ref.LlamaRef(cfg, host, f32_activations=True)
    for pos, tok in enumerate([3, 1000, 57]):
        nt, logits = model.decode(tok, pos)
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
        _, plogits, _ = plain.step(plain.embed(tok), pos)
        noise = rel(rlogits, plogits.astype(np.float64))
        assert 1e-3 < noise < 5e-2, noise  # what the Q8_0 activations cost: about a percent
        assert rel(logits, rlogits) <= noise, (pos, rel(logits, rlogits), noise)
        assert nt == int(np.argmax(logits))
    kptr, _, nbytes = model.kv_cache()
    kc = np.empty(nbytes // 4, np.float32)
    hip._check(hip.lib().candy_hip_d2h(dev.handle, kc.ctypes.data, kptr, nbytes))
    kc = kc.reshape(ref.k_cache.shape)
    assert rel(kc[0, :, :3], ref.k_cache[0, :, :3].astype(np.float64)) <= 1e-3


def test_decode_with_rows_too_long_for_the_batch1_kernels(dev):
    # FFN rows longer than the batch-1 kernels hold in registers (16640 > 8 x 64 units of 32 values): the down
    # projection takes the looping kernel into a buffer of its own and the residual is added afterwards.  A row of
    # 16640 re-quantized activations is where f32 summation order shows first (the op itself is 3e-7 from the CPU),
    # so the bar is the activation quantizer's noise, as above; the first step's first-layer k/v hold 1e-3.
    cfg = dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, head_dim=64, d_ffn=16640, vocab=256,
               max_pos=16, rms_eps=1e-5, rope_base=10000.0)
    fmts = {"default": synth.Q8_0, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    host, model = build(dev, cfg, fmts, seed=50)
    ref = llama_ref.LlamaRef(cfg, host)
    plain = llama_ref.LlamaRef(cfg, host, f32_activations=True)
    for pos, tok in enumerate([3, 200, 57]):
        nt, logits = model.decode(tok, pos)
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
        _, plogits, _ = plain.step(plain.embed(tok), pos)
        noise = rel(rlogits, plogits.astype(np.float64))
        assert rel(logits, rlogits) <= max(1e-3, 0.5 * noise), (pos, rel(logits, rlogits), noise)
        assert nt == int(np.argmax(logits))
    kptr, _, nbytes = model.kv_cache()
    kc = np.empty(nbytes // 4, np.float32)
    hip._check(hip.lib().candy_hip_d2h(dev.handle, kc.ctypes.data, kptr, nbytes))
    kc = kc.reshape(ref.k_cache.shape)
    assert rel(kc[0, :, :1], ref.k_cache[0, :, :1].astype(np.float64)) <= 1e-3


def test_full_depth_7b_step_within_activation_noise(dev):
    # The benchmark's model as configured: 32 layers 4096 / 11008, 32 heads x 128, vocab 32000, every matrix
    # N(0, 0.02) quantized on the device (one draw per shape, blocks rotated per layer), KV cache pre-filled with
    # N(0, 1) for 2048 positions.  One decode step on the device, as the CPU composition, and as the CPU composition
    # again with every Linear adding its blocks in another order (two of them).  By this depth correct evaluations
    # have drifted apart through rounding flips of the repeated Q8_0 re-quantization (tests/test_oracle_drift.py
    # measures that without a GPU), so the bar is taken from the CPU alone: the device may be no further from the
    # CPU composition than 1.5 times the distance between CPU evaluations of different summation order.  It must
    # also stay nearer to the CPU composition than that is to the model without the activation quantizer, and all
    # evaluations pick the same token.  About a minute, nearly all of it the CPU passes.
    n_layers, n_pos = 32, 2048
    cfg = dict(n_layers=n_layers, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=11008, vocab=32000,
               max_pos=n_pos + 8, rms_eps=1e-5, rope_base=10000.0)
    shapes = {"q": (4096, 4096), "k": (4096, 4096), "v": (4096, 4096), "o": (4096, 4096), "gate": (11008, 4096),
              "up": (11008, 4096), "down": (4096, 11008)}

    def drawn(fmt, r, k, seed):
        x = np.random.Generator(np.random.Philox(seed)).standard_normal((r, k), dtype=np.float32) * np.float32(0.02)
        return dev.quantize(fmt, x)

    base = {rk: drawn(synth.Q4_K, rk[0], rk[1], 100 + rk[0] + rk[1]).reshape(-1, 144) for rk in set(shapes.values())}
    host, model, shift = {}, hip.Llama(dev, **cfg), 0
    ones = np.ones(4096, np.float32)
    for l in range(n_layers):
        for kind, (r, k) in shapes.items():
            shift += 1
            b = np.roll(base[(r, k)], 977 * shift, axis=0).reshape(-1)
            host[(kind, l)] = (synth.Q4_K, b)
            model.set_qweight(KINDS[kind], l, dev.qtensor(synth.Q4_K, r, k, b))
        for kind in ("attn_norm", "ffn_norm"):
            host[(kind, l)] = ones
            model.set_norm(KINDS[kind], l, ones)
    host[("out_norm", -1)] = ones
    model.set_norm(hip.W_OUT_NORM, -1, ones)
    for kind, fmt, seed in (("head", synth.Q6_K, 7), ("embed", synth.Q8_0, 8)):
        b = drawn(fmt, 32000, 4096, seed)
        host[(kind, -1)] = (fmt, b)
        model.set_qweight(KINDS[kind], -1, dev.qtensor(fmt, 32000, 4096, b))
    # one pair of cache arrays shared by the CPU evaluations (1 GB each; each writes only the new position)
    rng = np.random.Generator(np.random.Philox(9))
    kptr, vptr, _ = model.kv_cache()
    caches = []
    for ptr in (kptr, vptr):
        full = np.zeros((n_layers, 32, cfg["max_pos"], 128), np.float32)
        full[:, :, :n_pos] = rng.standard_normal((n_layers, 32, n_pos, 128), dtype=np.float32)
        hip._check(hip.lib().candy_hip_h2d(dev.handle, ptr, full.ctypes.data, full.nbytes))
        caches.append(full)
    tok, pos = 1234, n_pos
    nt, logits = model.decode(tok, pos)

    def cpu(**kw):
        ref = llama_ref.LlamaRef(dict(cfg, max_pos=1), host, **kw)  # no cache of its own
        ref.c = cfg
        ref.k_cache, ref.v_cache = caches
        ref.cos, ref.sin = llama_ref.rope_tables(cfg["max_pos"], 128, cfg["rope_base"])
        t, lg, _ = ref.step(ref.embed(tok), pos)
        return t, lg.astype(np.float64)

    rt, rlogits = cpu()
    alts = [cpu(block_order=k) for k in (1, 2)]
    pt, plogits = cpu(f32_activations=True)
    drift = max(rel(a[1], rlogits) for a in alts)
    noise = rel(rlogits, plogits)
    err = rel(logits, rlogits)
    print(f"device vs CPU {err:.2e}; CPU vs CPU in another summation order {[round(rel(a[1], rlogits), 4) for a in alts]}; "
          f"CPU vs CPU without the activation quantizer {noise:.2e}")
    assert 5e-3 < drift < 0.2, drift
    assert err <= 1.5 * drift, (err, drift)
    assert err <= noise and rel(logits, plogits) <= 1.25 * noise, (err, noise)
    assert nt == rt == pt and all(a[0] == rt for a in alts)
    model.free()


def test_full_depth_7b_half_layers_teacher_forced(dev):
    # The benchmark's model again (32 layers 4096 / 11008, every matrix N(0, 0.02) quantized on the device, 2048 cached
    # positions of N(0, 1)), held to the per-op bar at every layer.  The CPU composition runs the whole step once and
    # records the hidden state in front of every layer and between its two halves.  The device then runs each HALF
    # layer on its own from the CPU's input for it - a one-layer model with that layer's weights and cache rows whose
    # other half is switched off with all-zero weights (zero FFN: the output is h + Wo.att; zero Wo: the attention
    # adds nothing and the output is h + Wdown.act) - and its k / v rows and output must match the CPU's to 1e-3.
    # A half layer is the longest stretch this bar can be asked of: it re-quantizes twice (norm output, then the
    # attention output or SiLU*Mul), a last-place difference may flip a rounding at the second quantizer, and with no
    # third quantizer behind it that moves the output by a few 1e-4 at most.  A whole layer has a third and fourth, where such a
    # flip is amplified to several 1e-3 (CPU evaluations in another summation order differ as much): the drift the
    # end-to-end test allows for.  Here it cannot hide a wrong layer.
    n_layers, n_pos = 32, 2048
    cfg = dict(n_layers=n_layers, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=11008, vocab=256,
               max_pos=n_pos + 8, rms_eps=1e-5, rope_base=10000.0)
    shapes = {"q": (4096, 4096), "k": (4096, 4096), "v": (4096, 4096), "o": (4096, 4096), "gate": (11008, 4096),
              "up": (11008, 4096), "down": (4096, 11008)}

    def drawn(fmt, r, k, seed):
        x = np.random.Generator(np.random.Philox(seed)).standard_normal((r, k), dtype=np.float32) * np.float32(0.02)
        return dev.quantize(fmt, x)

    base = {rk: drawn(synth.Q4_K, rk[0], rk[1], 300 + rk[0] + rk[1]).reshape(-1, 144) for rk in set(shapes.values())}
    rng = np.random.default_rng(17)
    host, qts, shift = {}, {}, 0
    for l in range(n_layers):
        for kind, (r, k) in shapes.items():
            shift += 1
            b = np.roll(base[(r, k)], 977 * shift, axis=0).reshape(-1)
            host[(kind, l)] = (synth.Q4_K, b)
            qts[(kind, l)] = dev.qtensor(synth.Q4_K, r, k, b)
        for kind in ("attn_norm", "ffn_norm"):
            host[(kind, l)] = (1 + 0.1 * rng.standard_normal(4096)).astype(np.float32)
    zero = {kind: dev.qtensor(synth.Q4_K, r, k, np.zeros(synth.weight_nbytes(synth.Q4_K, r, k), np.uint8))
            for kind, (r, k) in shapes.items() if kind in ("o", "gate", "up", "down")}
    host[("out_norm", -1)] = np.ones(4096, np.float32)
    for kind, fmt, seed in (("head", synth.Q6_K, 7), ("embed", synth.Q8_0, 8)):
        host[(kind, -1)] = (fmt, drawn(fmt, cfg["vocab"], 4096, seed))
    # CPU: one full step with a trace
    crng = np.random.Generator(np.random.Philox(19))
    ref = llama_ref.LlamaRef(dict(cfg, max_pos=1), host)
    ref.c = cfg
    ref.k_cache = np.zeros((n_layers, 32, cfg["max_pos"], 128), np.float32)
    ref.v_cache = np.zeros_like(ref.k_cache)
    ref.k_cache[:, :, :n_pos] = crng.standard_normal((n_layers, 32, n_pos, 128), dtype=np.float32)
    ref.v_cache[:, :, :n_pos] = crng.standard_normal((n_layers, 32, n_pos, 128), dtype=np.float32)
    ref.cos, ref.sin = llama_ref.rope_tables(cfg["max_pos"], 128, cfg["rope_base"])
    trace = []
    ref.step(ref.embed(77), n_pos, trace=trace)
    assert len(trace) == 2 * n_layers + 1
    # device: half a layer at a time from the CPU's inputs
    one = hip.Llama(dev, **dict(cfg, n_layers=1))
    one.set_norm(hip.W_OUT_NORM, -1, host[("out_norm", -1)])
    for kind in ("head", "embed"):
        fmt, b = host[(kind, -1)]
        one.set_qweight(KINDS[kind], -1, dev.qtensor(fmt, cfg["vocab"], 4096, b))
    kptr, vptr, nbytes = one.kv_cache()
    worst = {"k": 0.0, "v": 0.0, "attention half": 0.0, "ffn half": 0.0}
    for l in range(n_layers):
        for kind in ("attn_norm", "ffn_norm"):
            one.set_norm(KINDS[kind], 0, host[(kind, l)])
        for ptr, cache in ((kptr, ref.k_cache), (vptr, ref.v_cache)):
            rows = cache[l].copy()
            rows[:, n_pos] = 0  # the row this step writes
            hip._check(hip.lib().candy_hip_h2d(dev.handle, ptr, rows.ctypes.data, rows.nbytes))
        # attention half: the feed-forward weights are zero
        for kind in shapes:
            one.set_qweight(KINDS[kind], 0, zero[kind] if kind in ("gate", "up", "down") else qts[(kind, l)])
        one.decode_hidden(trace[2 * l], n_pos, want_logits=False)
        h_mid = one.hidden()
        kc, vc = read_cache(dev, one, (1, 32, cfg["max_pos"], 128))
        errs = {"k": rel(kc[0, :, n_pos], ref.k_cache[l, :, n_pos].astype(np.float64)),
                "v": rel(vc[0, :, n_pos], ref.v_cache[l, :, n_pos].astype(np.float64)),
                "attention half": rel(h_mid, trace[2 * l + 1].astype(np.float64))}
        assert np.array_equal(kc[0, :, :n_pos], ref.k_cache[l, :, :n_pos])  # nothing but the new row was touched
        # feed-forward half: Wo is zero, so the hidden state reaches the FFN as it was given
        for kind in shapes:
            one.set_qweight(KINDS[kind], 0, zero[kind] if kind == "o" else qts[(kind, l)])
        one.decode_hidden(trace[2 * l + 1], n_pos, want_logits=False)
        errs["ffn half"] = rel(one.hidden(), trace[2 * l + 2].astype(np.float64))
        for key, e in errs.items():
            worst[key] = max(worst[key], e)
            assert e <= 1e-3, (l, key, e)
    print("teacher-forced half layers, worst over 32 layers: " + ", ".join(f"{k} {v:.2e}" for k, v in worst.items()))
    one.free()
    for q in list(qts.values()) + list(zero.values()):
        q.free()


def test_full_depth_llama3_8b_shape_step(dev):
    # The Llama-3-8B-shaped model of the benchmark at full depth: 32 layers, 32 query / 8 kv heads x 128, d_ffn 14336,
    # vocab 128256, Q4_K attention and gate / up, Q6_K down (K = 14336 on the batch-1 kernel of its own) and head (the
    # norm launch + batch-1 path of a vocabulary-sized Q6_K head), Q8_0 embedding rows; 512 cached positions of
    # N(0, 1), one decode step from an embedding row.  The bar is the one the 7B step has: no further from the CPU
    # composition than 1.5 times the distance between CPU evaluations that add each row's blocks in another order
    # (or 1e-3 where that is larger), and the same token picked by all of them.
    n_layers, n_pos = 32, 512
    cfg = dict(n_layers=n_layers, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ffn=14336, vocab=128256,
               max_pos=n_pos + 8, rms_eps=1e-5, rope_base=500000.0)
    fmts = {"default": synth.Q4_K, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    host, model = build(dev, cfg, fmts, seed=88)
    rng = np.random.Generator(np.random.Philox(89))
    kptr, vptr, _ = model.kv_cache()
    caches = []
    for ptr in (kptr, vptr):
        full = np.zeros((n_layers, 8, cfg["max_pos"], 128), np.float32)
        full[:, :, :n_pos] = rng.standard_normal((n_layers, 8, n_pos, 128), dtype=np.float32)
        hip._check(hip.lib().candy_hip_h2d(dev.handle, ptr, full.ctypes.data, full.nbytes))
        caches.append(full)
    tok, pos = 100000, n_pos
    nt, logits = model.decode(tok, pos)

    def cpu(**kw):
        ref = llama_ref.LlamaRef(dict(cfg, max_pos=1), host, **kw)
        ref.c = cfg
        ref.k_cache, ref.v_cache = caches
        ref.cos, ref.sin = llama_ref.rope_tables(cfg["max_pos"], 128, cfg["rope_base"])
        t, lg, _ = ref.step(ref.embed(tok), pos)
        return t, lg.astype(np.float64)

    rt, rlogits = cpu()
    alts = [cpu(block_order=k) for k in (1, 2)]
    drift = max(rel(a[1], rlogits) for a in alts)
    err = rel(logits, rlogits)
    print(f"8B shape: device vs CPU {err:.2e}; CPU vs CPU in another summation order {[float('%.2e' % rel(a[1], rlogits)) for a in alts]}")
    assert err <= max(1e-3, 1.5 * drift), (err, drift)
    assert nt == int(np.argmax(logits))
    top2 = np.sort(rlogits)[-2:]
    if top2[1] - top2[0] > 2 * max(err, drift) * np.max(np.abs(rlogits)):
        assert nt == rt and all(a[0] == rt for a in alts)
    # the new k / v rows of the first layer (one quantizer upstream) hold the per-op bar
    kc, vc = read_cache(dev, model, (n_layers, 8, cfg["max_pos"], 128))
    assert rel(kc[0, :, pos], caches[0][0, :, pos].astype(np.float64)) <= 1e-3
    assert rel(vc[0, :, pos], caches[1][0, :, pos].astype(np.float64)) <= 1e-3
    model.free()


@pytest.mark.parametrize("d_ffn", [11008, 14336, 18432, 22016])
def test_long_cache_step_on_the_even_split_kernels(dev, d_ffn):
    # One full-width 7B layer over a cache of 600 positions with q/k/v and gate/up on the kernels that deal the rows
    # evenly over the CUs (two workgroups of eight wavefronts per CU, or one of sixteen; the wider FFNs give a
    # wavefront four, five and six row pairs, the fourth and later ones loaded into the registers of pairs already
    # contracted), against the CPU composition and against the same step on the narrower kernels (the RMS sum runs
    # in another order, so not the same bits).
    n_pos = 600
    cfg = dict(n_layers=1, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=d_ffn, vocab=512,
               max_pos=n_pos + 8, rms_eps=1e-5, rope_base=10000.0)
    fmts = {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    host, model = build(dev, cfg, fmts, seed=91)
    ref = llama_ref.LlamaRef(cfg, host)
    rng = np.random.Generator(np.random.Philox(92))
    kptr, vptr, _ = model.kv_cache()
    for name, ptr in (("k_cache", kptr), ("v_cache", vptr)):
        full = np.zeros((1, 32, cfg["max_pos"], 128), np.float32)
        full[:, :, :n_pos] = rng.standard_normal((1, 32, n_pos, 128), dtype=np.float32)
        getattr(ref, name)[:] = full
        hip._check(hip.lib().candy_hip_h2d(dev.handle, ptr, full.ctypes.data, full.nbytes))
    tok = 77
    rt, rlogits, _ = ref.step(ref.embed(tok), n_pos)
    results = {}
    try:
        for wide, waves in ((1, 8), (1, 16), (0, 8)):
            dev.set_option("fused.wide", wide)
            dev.set_option("fused.wide_waves", waves)
            model.set_graph(True)  # captured again under the new options
            nt, logits = model.decode(tok, n_pos)
            assert rel(logits, rlogits) <= 1e-3, (wide, waves, rel(logits, rlogits))
            assert nt == int(np.argmax(logits))
            results[(wide, waves)] = logits
            nt2, again = model.decode(tok, n_pos)  # a second replay: the same bits (tickets back at zero)
            assert np.array_equal(logits, again)
    finally:
        dev.set_option("fused.wide", 1)
        dev.set_option("fused.wide_waves", 8)
    assert rel(results[(1, 8)], results[(0, 8)].astype(np.float64)) <= 1e-3
    assert rel(results[(1, 16)], results[(0, 8)].astype(np.float64)) <= 1e-3
    kc, vc = read_cache(dev, model, ref.k_cache.shape)
    assert rel(kc[:, :, n_pos], ref.k_cache[:, :, n_pos].astype(np.float64)) <= 1e-3
    model.free()


PROMPT_CASES = [
    # (name, cfg, formats, prompt length, bar): lengths on both sides of the 16-row switch to MFMA tiles
    # and off the 32-query attention tile. Q4_K and Q6_K tiles are integer-exact, so the prompt pass
    # holds the decode step's 1e-3.
    ("gqa-q4k-q6k-down", dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=2, head_dim=64, d_ffn=1024, vocab=512,
                              max_pos=64, rms_eps=1e-5, rope_base=500000.0),
     {"default": synth.Q4_K, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}, 37, 1e-3),
    ("mha-hd128", dict(n_layers=2, d_model=512, n_heads=4, n_kv_heads=4, head_dim=128, d_ffn=768, vocab=256,
                       max_pos=80, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}, 70, 1e-3),
    ("gqa-hd128-long", dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=2, head_dim=128, d_ffn=512, vocab=256,
                            max_pos=224, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}, 203, 1e-3),
    ("other-formats", dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=4, head_dim=64, d_ffn=1024, vocab=256,
                           max_pos=32, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q5_K, "q": synth.Q5_0, "k": synth.Q4_1, "v": synth.Q5_1, "gate": synth.Q3_K, "up": synth.Q2_K,
      "head": synth.Q4_1_GGML, "embed": synth.Q8_K}, 21, 1e-3),  # every one of them on the integer-exact tiles
    ("short-prompt", dict(n_layers=2, d_model=256, n_heads=4, n_kv_heads=2, head_dim=64, d_ffn=512, vocab=128,
                          max_pos=16, rms_eps=1e-5, rope_base=10000.0),
     {"default": synth.Q8_0, "gate": synth.Q4_0, "head": synth.Q6_K, "embed": synth.Q4_K}, 5, 1e-3),
]


@pytest.mark.parametrize("name,cfg,fmts,n,bar", PROMPT_CASES)
def test_prompt_pass_matches_token_by_token_cpu(dev, name, cfg, fmts, n, bar):
    host, model = build(dev, cfg, fmts, seed=11)
    ref = llama_ref.LlamaRef(cfg, host)
    rng = np.random.default_rng(12)
    tokens = [int(t) for t in rng.integers(0, cfg["vocab"], n)]
    for pos, tok in enumerate(tokens):  # the CPU composition has no batched form: token by token
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
    nt, logits = model.prefill(tokens, 0)
    assert rel(logits, rlogits) <= bar, name
    assert nt == int(np.argmax(logits))
    kptr, vptr, nbytes = model.kv_cache()
    for ptr, want in ((kptr, ref.k_cache), (vptr, ref.v_cache)):
        got = np.empty(nbytes // 4, np.float32)
        hip._check(hip.lib().candy_hip_d2h(dev.handle, got.ctypes.data, ptr, nbytes))
        got = got.reshape(want.shape)
        assert rel(got[:, :, :n], want[:, :, :n].astype(np.float64)) <= bar
        assert not got[:, :, n:].any()  # nothing written past the prompt
    # decoding continues from the cache the prompt pass left
    tok = nt
    for pos in range(n, n + 3):
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
        gt, glogits = model.decode(tok, pos)
        assert rel(glogits, rlogits) <= bar, (name, pos)
        tok = rt


BIG_PROMPT_CFG = dict(n_layers=2, d_model=512, n_heads=8, n_kv_heads=2, head_dim=128, d_ffn=1536, vocab=512,
                      max_pos=520, rms_eps=1e-5, rope_base=500000.0)
BIG_PROMPT_FMTS = {"default": synth.Q4_K, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}


@pytest.mark.parametrize("n", [256, 300, 512])
def test_prompt_pass_of_256_rows_and_more_matches_cpu(dev, n):
    # From 256 rows on every Linear of the prompt pass contracts fp16 operands (the dequantized weight and d * q of
    # the Q8_0 activations, each rounded once to fp16) on the big tiles, the kernels that quantize an activation also
    # write its fp16 expansion, and residual adds ride in the projection's epilogue or in the sum over the K splits.
    # Checked against the CPU composition (integer dots) token by token; what the operand rounding costs end to
    # end is measured on the CPU alone, as the same composition with fp16 operands against the exact one, and the
    # device has to stay within 1.5 times that (or within 1e-3 where that is larger).
    cfg, fmts = BIG_PROMPT_CFG, BIG_PROMPT_FMTS
    host, model = build(dev, cfg, fmts, seed=71)
    tokens = [int(t) for t in np.random.default_rng(72 + n).integers(0, cfg["vocab"], n)]
    exact = llama_ref.LlamaRef(cfg, host)
    et, elogits, _ = exact.prefill(tokens)
    rounded = llama_ref.LlamaRef(cfg, host, fp16_operands=True)
    _, rlogits, _ = rounded.prefill(tokens)
    noise = rel(rlogits, elogits.astype(np.float64))
    nt, logits = model.prefill(tokens, 0)
    err = rel(logits, elogits.astype(np.float64))
    print(f"n={n}: device vs exact CPU {err:.2e}; fp16-operand CPU vs exact CPU {noise:.2e}; "
          f"device vs fp16-operand CPU {rel(logits, rlogits.astype(np.float64)):.2e}")
    assert err <= max(1e-3, 1.5 * noise), (n, err, noise)
    assert nt == int(np.argmax(logits))
    kc, vc = read_cache(dev, model, exact.k_cache.shape)
    # the first layer's k / v are one fp16-operand Linear away from the embedding rows: the per-matmul bar
    assert rel(kc[0, :, :n], exact.k_cache[0, :, :n].astype(np.float64)) <= 1e-3
    assert rel(vc[0, :, :n], exact.v_cache[0, :, :n].astype(np.float64)) <= 1e-3
    # deeper layers' k / v: held against what the operand rounding does to the same arrays on the CPU
    for got, want, rnd in ((kc, exact.k_cache, rounded.k_cache), (vc, exact.v_cache, rounded.v_cache)):
        cache_noise = rel(rnd[:, :, :n], want[:, :, :n].astype(np.float64))
        assert rel(got[:, :, :n], want[:, :, :n].astype(np.float64)) <= max(1e-3, 1.5 * cache_noise), (n, cache_noise)
        assert not got[:, :, n:].any()
    # decoding continues from the cache the prompt pass left; the CPU continues from its own, and the rounded
    # composition from its rounded cache says how much of the difference the cache carries over
    tok = nt
    for pos in range(n, n + 2):
        rt, slogits, _ = exact.step(exact.embed(tok), pos)
        _, nlogits, _ = rounded.step(rounded.embed(tok), pos)
        gt, glogits = model.decode(tok, pos)
        step_noise = max(noise, rel(nlogits, slogits.astype(np.float64)))
        assert rel(glogits, slogits.astype(np.float64)) <= max(1e-3, 1.5 * step_noise), (n, pos, step_noise)
        tok = rt


WIDE_PROMPT_CFG = dict(n_layers=2, d_model=5120, n_heads=8, n_kv_heads=2, head_dim=128, d_ffn=1024, vocab=256,
                       max_pos=300, rms_eps=1e-5, rope_base=10000.0)


@pytest.mark.parametrize("n,wide", [(64, False), (256, False), (300, False), (512, False), (272, True)])
def test_split_sums_inside_the_following_launch_equal_separate_launches(dev, n, wide):
    # A projection that splits K hands its partial copies to the launch behind it: o / down to the RMSNorm + quantize
    # launch (the last layer's down projection to a split sum of its own), the q / k / v grid to the rope launch.
    # Same additions in the same order as the separate split sum, residual add, norm and rope: every cached k / v
    # and the logits the same bits.  `wide`: hidden rows of 5120 values (the norm launch then holds eight vectors a thread,
    # five of them live).
    cfg, fmts = (WIDE_PROMPT_CFG if wide else BIG_PROMPT_CFG), BIG_PROMPT_FMTS
    _, a = build(dev, cfg, fmts, seed=72)
    _, b = build(dev, cfg, fmts, seed=72)
    tokens = [int(t) for t in np.random.default_rng(190 + n).integers(0, cfg["vocab"], n)]
    ta, la = a.prefill(tokens, 0)
    dev.set_option("prefill.fold_split_sums", 0)
    try:
        tb, lb = b.prefill(tokens, 0)
    finally:
        dev.set_option("prefill.fold_split_sums", 1)
    shape = (cfg["n_layers"], cfg["n_kv_heads"], cfg["max_pos"], cfg["head_dim"])
    ka, va = read_cache(dev, a, shape)
    kb, vb = read_cache(dev, b, shape)
    assert np.array_equal(ka.view(np.uint32), kb.view(np.uint32))
    assert np.array_equal(va.view(np.uint32), vb.view(np.uint32))
    assert np.array_equal(la.view(np.uint32), lb.view(np.uint32)) and ta == tb


@pytest.mark.parametrize("n", [256, 300, 512])
def test_grouped_qkv_projection_agrees_with_separate_launches(dev, n):
    # From 256 rows on the q / k / v projections share one grid of fp16 tiles (their outputs lie end to end, one sum
    # over the K splits serves the three).  The same tiles one projection per launch split K differently, so the two
    # agree to f32 summation order, not bit for bit: first-layer k / v within 1e-5, logits within 1e-4.
    cfg, fmts = BIG_PROMPT_CFG, BIG_PROMPT_FMTS
    _, a = build(dev, cfg, fmts, seed=71)
    _, b = build(dev, cfg, fmts, seed=71)
    tokens = [int(t) for t in np.random.default_rng(90 + n).integers(0, cfg["vocab"], n)]
    ta, la = a.prefill(tokens, 0)
    dev.set_option("prefill.qkv_group", 0)
    try:
        tb, lb = b.prefill(tokens, 0)
    finally:
        dev.set_option("prefill.qkv_group", 1)
    shape = (cfg["n_layers"], cfg["n_kv_heads"], cfg["max_pos"], cfg["head_dim"])
    ka, va = read_cache(dev, a, shape)
    kb, vb = read_cache(dev, b, shape)
    assert rel(ka[0, :, :n], kb[0, :, :n].astype(np.float64)) <= 1e-5
    assert rel(va[0, :, :n], vb[0, :, :n].astype(np.float64)) <= 1e-5
    assert not ka[:, :, n:].any() and not va[:, :, n:].any()
    assert rel(la, lb.astype(np.float64)) <= 1e-4
    assert ta == tb


def test_full_width_prompt_pass_of_256_rows(dev):
    # One layer at the Llama-3-8B width (d_model 4096, 32 query / 8 kv heads x 128, d_ffn 14336, Q4_K with a Q6_K
    # down projection), 256 tokens: the shapes and kernels of the benchmark's prompt pass (fp16 big tiles, K split
    # over workgroups for the narrow k / v projections, residual in the epilogue), against the CPU composition.
    cfg = dict(n_layers=1, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ffn=14336, vocab=512,
               max_pos=264, rms_eps=1e-5, rope_base=500000.0)
    fmts = {"default": synth.Q4_K, "down": synth.Q6_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    n = 256
    host, model = build(dev, cfg, fmts, seed=81)
    tokens = [int(t) for t in np.random.default_rng(82).integers(0, cfg["vocab"], n)]
    exact = llama_ref.LlamaRef(cfg, host)
    _, elogits, _ = exact.prefill(tokens)
    rounded = llama_ref.LlamaRef(cfg, host, fp16_operands=True)
    _, rlogits, _ = rounded.prefill(tokens)
    noise = rel(rlogits, elogits.astype(np.float64))
    nt, logits = model.prefill(tokens, 0)
    err = rel(logits, elogits.astype(np.float64))
    print(f"full width: device vs exact CPU {err:.2e}; fp16-operand CPU vs exact CPU {noise:.2e}")
    assert err <= max(1e-3, 1.5 * noise), (err, noise)
    kc, vc = read_cache(dev, model, exact.k_cache.shape)
    assert rel(kc[0, :, :n], exact.k_cache[0, :, :n].astype(np.float64)) <= 1e-3
    assert rel(vc[0, :, :n], exact.v_cache[0, :, :n].astype(np.float64)) <= 1e-3
    model.free()


def read_cache(dev, model, shape):
    """Both device caches as f32 arrays, whichever element type they hold."""
    kptr, vptr, nbytes = model.kv_cache()
    n = int(np.prod(shape))
    dt = {4 * n: np.float32, 2 * n: np.float16}[nbytes]
    out = []
    for ptr in (kptr, vptr):
        got = np.empty(n, dt)
        hip._check(hip.lib().candy_hip_d2h(dev.handle, got.ctypes.data, ptr, nbytes))
        out.append(got.astype(np.float32).reshape(shape))
    return out


@pytest.mark.parametrize("layers", [1, 2])
@pytest.mark.parametrize("case", [0, 1, 2])
def test_fp16_kv_cache_matches_cpu_composition_with_rounded_cache(dev, case, layers):
    # The optional half-size cache: k and v rounded to fp16 once, on entry; the CPU composition rounds the same
    # values the same way.
    # One layer: k and v come straight from the first projections, device and CPU agree to 1e-7 before rounding,
    # nearly every stored number is the same fp16 value, and the f32 cache's 1e-3 bar holds as it is.
    # Two layers: the second layer's k and v are 1e-4 apart before rounding, one value in ten straddles an fp16
    # rounding boundary and is stored a whole fp16 step apart, so the two runs differ by a fraction of the noise
    # the rounding itself adds.  That noise is measured here (CPU composition with the rounded cache against the
    # same with candy's f32 cache; large on these random-block models, whose softmax is close to an argmax) and is
    # the bar wherever it exceeds 1e-3.
    # Cases: head_dim 64 (vector-ALU prompt attention, GQA), head_dim 128 MHA and GQA (matrix-core prompt
    # attention), decode continuing from each.
    name, cfg, fmts, n, bar = PROMPT_CASES[case]
    cfg = dict(cfg, n_layers=layers)
    host, model = build(dev, cfg, fmts, seed=21)
    model.set_kv_f16(True)
    ref = llama_ref.LlamaRef(cfg, host, kv_f16=True)
    plain = llama_ref.LlamaRef(cfg, host)
    tokens = [int(t) for t in np.random.default_rng(22).integers(0, cfg["vocab"], n)]

    def cpu_step(tok, pos, strict=layers == 1):
        rt, rlogits, _ = ref.step(ref.embed(tok), pos)
        _, plogits, _ = plain.step(plain.embed(tok), pos)
        noise = rel(rlogits, plogits.astype(np.float64))
        return rt, rlogits, bar if strict else max(bar, noise)

    for pos, tok in enumerate(tokens):
        rt, rlogits, lim = cpu_step(tok, pos)
    nt, logits = model.prefill(tokens, 0)
    assert rel(logits, rlogits) <= lim, name
    assert model.kv_cache()[2] == ref.k_cache.size * 2
    for got, want in zip(read_cache(dev, model, ref.k_cache.shape), (ref.k_cache, ref.v_cache)):
        assert rel(got[:, :, :n], want[:, :, :n].astype(np.float64)) <= bar + 2.0 ** -10  # one fp16 step more
        assert np.mean(got[:, :, :n] == want[:, :, :n]) > 0.8  # and most are the same fp16 number
        assert np.mean(got[0, :, :n] == want[0, :, :n]) > 0.99  # the first layer's, all but stray straddles
        assert not got[:, :, n:].any()
    tok = nt
    for pos in range(n, n + 3):
        rt, rlogits, lim = cpu_step(tok, pos)
        gt, glogits = model.decode(tok, pos)
        assert rel(glogits, rlogits) <= lim, (name, pos)
        tok = rt
    # a short prompt (12 rows: one 16-row tile of the int8 kernel, whose sums run in another order than the batch-1
    # kernel's and the CPU's, so even the first layer's k and v straddle a rounding boundary here and there: the
    # rounding noise is the bar) and token by token from an empty cache both follow the CPU composition; switching
    # back to f32 clears the cache and restores candy's cache to the f32 bar
    _, other = build(dev, cfg, fmts, seed=21)
    other.set_kv_f16(True)
    ref, plain = llama_ref.LlamaRef(cfg, host, kv_f16=True), llama_ref.LlamaRef(cfg, host)
    for pos, t in enumerate(tokens[:12]):
        ot, ologits = other.decode(t, pos)
        rt, rlogits, lim = cpu_step(t, pos, strict=False)
    pt, plogits = model.prefill(tokens[:12], 0)
    assert rel(ologits, rlogits) <= lim
    assert rel(plogits, rlogits) <= lim
    model.set_kv_f16(False)
    assert model.kv_cache()[2] == ref.k_cache.size * 4
    assert not any(c.any() for c in read_cache(dev, model, ref.k_cache.shape))
    again = llama_ref.LlamaRef(cfg, host)
    for pos, t in enumerate(tokens[:6]):
        rt, rlogits, _ = again.step(again.embed(t), pos)
        gt, glogits = model.decode(t, pos)
    assert rel(glogits, rlogits) <= bar


def test_fp16_kv_cache_differs_from_f32_cache_by_its_rounding_only(dev):
    # how far the half-size cache moves the logits: well under the activation quantizer's own 1e-2, and not zero
    name, cfg, fmts, n, _ = PROMPT_CASES[1]
    host, a = build(dev, cfg, fmts, seed=23)
    _, b = build(dev, cfg, fmts, seed=23)
    b.set_kv_f16(True)
    tokens = [int(t) for t in np.random.default_rng(24).integers(0, cfg["vocab"], n)]
    _, la = a.prefill(tokens, 0)
    _, lb = b.prefill(tokens, 0)
    d = rel(lb, la.astype(np.float64))
    assert 0 < d < 1e-2, d


@pytest.mark.parametrize("case,n,cut", [(0, 50, 19), (2, 150, 77)])
def test_prompt_in_two_chunks_equals_one_pass(dev, case, n, cut):
    # a prompt continued at pos0 > 0 attends the positions already in the cache (head_dim 64: vector-ALU
    # attention; head_dim 128: the matrix-core kernel, second chunk starting off every tile boundary)
    name, cfg, fmts, _, _ = PROMPT_CASES[case]
    _, a = build(dev, cfg, fmts, seed=13)
    _, b = build(dev, cfg, fmts, seed=13)
    tokens = [int(t) for t in np.random.default_rng(14).integers(0, cfg["vocab"], n)]
    ta, la = a.prefill(tokens, 0)
    b.prefill(tokens[:cut], 0)
    tb, lb = b.prefill(tokens[cut:], cut)
    assert rel(lb, la.astype(np.float64)) <= 1e-4
    with pytest.raises(hip.CandyHipError, match="outside the cache"):
        a.prefill(tokens, cfg["max_pos"] - 10)
    with pytest.raises(hip.CandyHipError, match="empty"):
        a.prefill([], 0)


@pytest.mark.parametrize("cut", [20, 77, 128])
def test_prompt_attention_with_one_and_two_key_tile_groups(dev, cut):
    # The matrix-core kernel's two forms (one group of wavefronts per query tile walking every key tile; two groups
    # taking alternate tiles and merging at the end) agree on a whole prompt and on a chunk continued off the tile
    # boundaries: at pos0 = 20 the second group's first tile (keys 32..63) lies wholly in the future of some rows of a
    # wavefront that others of its rows can see.
    name, cfg, fmts, n, _ = PROMPT_CASES[2]
    tokens = [int(t) for t in np.random.default_rng(31).integers(0, cfg["vocab"], n)]
    got = {}
    try:
        for groups in (1, 2):
            dev.set_option("prefill.attention_groups", groups)
            _, a = build(dev, cfg, fmts, seed=30)
            _, b = build(dev, cfg, fmts, seed=30)
            _, whole = a.prefill(tokens, 0)
            b.prefill(tokens[:cut], 0)
            _, chunked = b.prefill(tokens[cut:], cut)
            assert rel(chunked, whole.astype(np.float64)) <= 1e-4, groups
            got[groups] = whole
    finally:
        dev.set_option("prefill.attention_groups", 0)
    assert rel(got[2], got[1].astype(np.float64)) <= 1e-5


def test_prompt_chunks_on_either_side_of_the_fp16_threshold(dev):
    # Results are not invariant under batching: a 300-token prompt fed whole contracts fp16 operands (256 rows or
    # more), the same prompt fed as 150 + 150 runs every Linear on the exact int8 kernels.  The two agree within
    # what the operand rounding costs end to end (measured on the CPU in the test above for this model: a few 1e-3),
    # not bit for bit; 255 and 256 tokens sit on either side of the threshold the same way.
    cfg, fmts = BIG_PROMPT_CFG, BIG_PROMPT_FMTS
    _, a = build(dev, cfg, fmts, seed=71)
    _, b = build(dev, cfg, fmts, seed=71)
    tokens = [int(t) for t in np.random.default_rng(372).integers(0, cfg["vocab"], 300)]
    ta, la = a.prefill(tokens, 0)
    b.prefill(tokens[:150], 0)
    tb, lb = b.prefill(tokens[150:], 150)
    d = rel(lb, la.astype(np.float64))
    print(f"300 tokens whole (fp16 operands) against 150 + 150 (int8): {d:.2e}")
    assert 0 < d <= 2e-2, d
    _, l255 = a.prefill(tokens[:255], 0)
    _, l256 = b.prefill(tokens[:256], 0)
    assert l255.shape == l256.shape  # the logits of the last token of each: different tokens, both finite
    assert np.isfinite(l255).all() and np.isfinite(l256).all()
    # the first 255 positions of the cache: exact kernels on one side, fp16 operands on the other, first layer 1e-3
    ka, _ = read_cache(dev, a, (cfg["n_layers"], cfg["n_kv_heads"], cfg["max_pos"], cfg["head_dim"]))
    kb, _ = read_cache(dev, b, (cfg["n_layers"], cfg["n_kv_heads"], cfg["max_pos"], cfg["head_dim"]))
    assert 0 < rel(kb[0, :, :255], ka[0, :, :255].astype(np.float64)) <= 1e-3


@pytest.mark.parametrize("d_ffn", [11008, 14336, 1024 + 256])
def test_gate_up_block_parts_give_the_same_bits(dev, d_ffn):
    # The narrower fused gate/up kernel (fused.wide = 0) lets a workgroup own a whole 32-value block of the FFN
    # activation or a half / quarter of one (whichever divides the rows evenly over the CUs); the block is quantized
    # from the same 32 f32 values either way, so the logits are the same bits, step after step (the per-block
    # counters return to zero).
    cfg = dict(n_layers=2, d_model=4096 if d_ffn > 4096 else 512, n_heads=8, n_kv_heads=8,
               head_dim=512 // 8 if d_ffn <= 4096 else 128, d_ffn=d_ffn, vocab=512, max_pos=16, rms_eps=1e-5, rope_base=10000.0)
    if d_ffn > 4096:
        cfg.update(n_heads=32, n_kv_heads=32)
    fmts = {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    tokens = [int(t) for t in np.random.default_rng(31).integers(0, cfg["vocab"], 5)]
    runs = {}
    dev.set_option("fused.wide", 0)
    try:
        for rows in ("32", "16", "8"):
            dev.set_option("fused.pair_rows", int(rows))
            _, model = build(dev, cfg, fmts, seed=30)
            runs[rows] = [model.decode(t, pos)[1].copy() for pos, t in enumerate(tokens)]
            model.free()
    finally:
        dev.set_option("fused.pair_rows", 0)
        dev.set_option("fused.wide", 1)
    for rows in ("16", "8"):
        for a, b in zip(runs["32"], runs[rows]):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), rows


@pytest.mark.parametrize("d_ffn", [11008, 14336])
def test_even_split_gate_up_hand_over_and_quantizing_down_projection_give_the_same_bits(dev, d_ffn):
    # The even-split gate/up kernel (fused.wide = 1) deals the row pairs to two or three workgroups per CU wherever
    # they fall, so most 32-value blocks of the FFN activation belong to two workgroups (d_ffn 11008: 512 workgroups
    # of 21.5 pairs; 14336: 512 of 28).  Two ways to get them quantized, same bits asked:
    #   fused.down_quant = 0  the parts of a block meet through write-through stores and a per-block ticket, the
    #                         workgroup that draws the last ticket quantizes (this rests on gfx950's memory behaviour,
    #                         not on the HIP memory model: this test is what covers it);
    #   fused.down_quant = 1  gate/up stores its f32 values and the down projection quantizes them in its prologue.
    # Twenty steps each, captured graph replayed, against each other and against one-by-one launches.
    cfg = dict(n_layers=2, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=d_ffn, vocab=512, max_pos=24,
               rms_eps=1e-5, rope_base=10000.0)
    fmts = {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    tokens = [int(t) for t in np.random.default_rng(33).integers(0, cfg["vocab"], 20)]
    runs = {}
    try:
        for key, down_quant, graph in (("tickets", 0, True), ("quantizing down", 1, True), ("tickets, eager", 0, False)):
            dev.set_option("fused.down_quant", down_quant)
            _, model = build(dev, cfg, fmts, seed=34)
            model.set_graph(graph)
            runs[key] = [model.decode(t, pos)[1].copy() for pos, t in enumerate(tokens)]
            model.free()
    finally:
        dev.set_option("fused.down_quant", 0)
    for key in ("quantizing down", "tickets, eager"):
        for pos, (a, b) in enumerate(zip(runs["tickets"], runs[key])):
            assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (key, pos)


def test_graph_replay_equals_eager_launches(dev):
    # the captured step is replayed for every token; every replay must give what one-by-one
    # launches give, with other work and synchronisations in between
    cfg = dict(n_layers=2, d_model=1024, n_heads=8, n_kv_heads=4, head_dim=128, d_ffn=2816, vocab=1024, max_pos=12,
               rms_eps=1e-5, rope_base=10000.0)
    fm = {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    _, eager = build(dev, cfg, fm, seed=9)
    _, graph = build(dev, cfg, fm, seed=9)
    eager.set_graph(False)
    tokens = [5, 900, 17, 17, 3, 64, 1000, 2]
    for pos, tok in enumerate(tokens):
        et, el = eager.decode(tok, pos)
        gt, gl = graph.decode(tok, pos)
        assert np.array_equal(el, gl), pos
        assert et == gt
        # unrelated work on the same device between replays
        dev.softmax(np.arange(64, dtype=np.float32), 64)
        dev.synchronize()


def test_generate_chains_the_same_tokens_as_step_by_step_decoding(dev):
    # candy_hip_llama_generate hands each step's greedy token to the next step in device memory and copies the list
    # out once; the tokens are those of candy_hip_llama_decode called step by step (graph replay and one-by-one
    # launches), and the cache ends up the same.
    cfg = dict(n_layers=2, d_model=1024, n_heads=8, n_kv_heads=4, head_dim=128, d_ffn=2816, vocab=1024, max_pos=24,
               rms_eps=1e-5, rope_base=10000.0)
    fmts = {"default": synth.Q4_K, "head": synth.Q6_K, "embed": synth.Q8_0}
    _, model = build(dev, cfg, fmts, seed=77, from_normal=True)  # such weights do not settle on one token at once
    n = 12
    for graph in (True, False):
        model.set_graph(graph)
        tok, steps = 3, []
        for pos in range(n):
            tok, _ = model.decode(tok, pos, want_logits=False)
            steps.append(tok)
        k_steps, v_steps = read_cache(dev, model, (cfg["n_layers"], cfg["n_kv_heads"], cfg["max_pos"], cfg["head_dim"]))
        chained = model.generate(3, 0, n)
        assert chained == steps, (graph, chained, steps)
        k_gen, v_gen = read_cache(dev, model, (cfg["n_layers"], cfg["n_kv_heads"], cfg["max_pos"], cfg["head_dim"]))
        assert np.array_equal(k_steps[:, :, :n], k_gen[:, :, :n]) and np.array_equal(v_steps[:, :, :n], v_gen[:, :, :n])
        assert len(set(steps)) > 1  # the chain is not a fixed point from the first token on
    # a single step, and one more from where the list ended
    assert model.generate(3, 0, 1) == steps[:1]
    with pytest.raises(hip.CandyHipError):
        model.generate(3, cfg["max_pos"] - 2, 3)
    with pytest.raises(hip.CandyHipError):
        model.generate(cfg["vocab"], 0, 2)
    with pytest.raises(hip.CandyHipError):
        model.generate(3, 0, 0)
    model.free()


def test_greedy_token_over_several_workgroups_ties_and_an_odd_vocabulary(dev):
    # The decoder's argmax folds the logits of a long row into one word from several workgroups.  A vocabulary of 4099
    # (two workgroups of 16-byte pieces + three trailing values) whose head rows are all the same block bytes gives 4099
    # bit-identical logits: the first index must win whichever workgroup arrives first.  With the last row's scales
    # negated (a value in the trailing part) and with a row in the second workgroup's part negated, the token is
    # numpy's argmax of the logits (first maximum) step after step, over replayed graphs and one-by-one launches.
    cfg = dict(n_layers=1, d_model=256, n_heads=2, n_kv_heads=2, head_dim=128, d_ffn=512, vocab=4099, max_pos=8,
               rms_eps=1e-5, rope_base=10000.0)
    fmts = {"default": synth.Q4_K, "head": synth.Q8_0, "embed": synth.Q8_0}
    host, model = build(dev, cfg, fmts, seed=88)
    fmt, blocks = host[("head", -1)]
    bb = synth.BLOCK_BYTES[fmt]
    rows = np.array(blocks, copy=True).reshape(cfg["vocab"], -1)
    rows[:] = rows[0]
    keep = []
    for variant in ("all equal", "last row negated", "a row of the second part negated"):
        r = rows.copy()
        if variant != "all equal":
            at = cfg["vocab"] - 1 if variant == "last row negated" else 3000
            r[at].reshape(-1, bb)[:, 1] ^= 0x80  # sign bit of every block's fp16 scale
        head = dev.qtensor(fmt, cfg["vocab"], cfg["d_model"], r.reshape(-1))
        keep.append(head)
        model.set_qweight(hip.W_HEAD, -1, head)
        for graph in (True, False):
            model.set_graph(graph)
            for pos, tok in enumerate([5, 4098, 77]):
                nt, logits = model.decode(tok, pos)
                assert nt == int(np.argmax(logits)), (variant, graph, pos, nt, int(np.argmax(logits)))
                if variant == "all equal":
                    assert np.all(logits.view(np.uint32) == logits.view(np.uint32)[0]) and nt == 0
            chained = model.generate(5, 0, 3)
            assert len(chained) == 3 and all(0 <= t < cfg["vocab"] for t in chained)
    # Logits that are NaN or -inf are never chosen (reduce.go:846-862 compares with a strict > against -MaxFloat32,
    # so a row of nothing else yields 0); +inf is.  Head rows with a NaN scale give NaN logits, rows with an infinite
    # scale +inf, -inf or NaN.
    def reference_choice(logits):
        best, at = np.float32(-3.4028234663852886e38), 0
        for i, v in enumerate(logits):
            if v > best:
                best, at = v, i
        return at
    _, plain = host[("head", -1)]
    base = np.array(plain, copy=True).reshape(cfg["vocab"], -1)
    for variant in ("every logit NaN", "NaN in front, finite behind", "infinite scales"):
        r = base.copy()
        blk = r.reshape(cfg["vocab"], -1, bb)
        if variant == "every logit NaN":
            blk[:, :, 0], blk[:, :, 1] = 0x00, 0x7E
        elif variant == "NaN in front, finite behind":
            blk[:700, :, 0], blk[:700, :, 1] = 0x00, 0x7E
        else:
            blk[1000:1100, :, 0], blk[1000:1100, :, 1] = 0x00, 0x7C
        head = dev.qtensor(fmt, cfg["vocab"], cfg["d_model"], r.reshape(-1))
        keep.append(head)
        model.set_qweight(hip.W_HEAD, -1, head)
        model.set_graph(True)
        for pos, tok in enumerate([5, 4098, 77]):
            nt, logits = model.decode(tok, pos)
            assert nt == reference_choice(logits), (variant, pos, nt, reference_choice(logits))
            if variant == "every logit NaN":
                assert np.all(np.isnan(logits)) and nt == 0
            if variant == "NaN in front, finite behind":
                assert np.all(np.isnan(logits[:700])) and nt >= 700
    model.free()


def test_decode_errors(dev):
    cfg = dict(n_layers=1, d_model=256, n_heads=2, n_kv_heads=2, head_dim=128, d_ffn=256, vocab=64, max_pos=4,
               rms_eps=1e-5, rope_base=10000.0)
    model = hip.Llama(dev, **cfg)
    with pytest.raises(hip.CandyHipError, match="embedding table not set"):
        model.decode(0, 0)
    with pytest.raises(hip.CandyHipError, match="must be"):
        model.set_qweight(hip.W_Q, 0, dev.qtensor(synth.Q4_K, 8, 256, synth.random_weight(synth.Q4_K, 8, 256, 1)))
    host, model = build(dev, cfg, {"default": synth.Q4_K}, seed=1)
    with pytest.raises(hip.CandyHipError, match="outside the cache"):
        model.decode(0, 4)
    with pytest.raises(hip.CandyHipError, match="outside the vocabulary"):
        model.decode(64, 0)
