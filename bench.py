#!/usr/bin/env python3
"""Benchmark of the quantized-matmul hot path on one MI355X.

`python bench.py --gpus 1 --steps K --warmup W` prints ONE JSON line.

Workload (the one the headline metric is quoted on): Q4_K weight 4096 x 11008
(N outputs x K contraction, 25 362 432 bytes of blocks), batch 1, f32 activation in, f32
output out.  A "step" is one pass of that path: quantize the activation to Q8_0 on the
device, then the matvec.  Steps rotate over enough distinct copies of the weight (>= 512 MB)
that none of it is still in the 256 MB last-level cache when it is read again, so `value` is
an HBM figure.  Inputs are resident in HBM before the timed region starts.

A timed "step" is ONE such call.  So that a short `--steps` still gives a steady figure, every step is
repeated `config.inner_reps` times back to back inside the timed region (at least 1000 timed calls in all) and
`ms_per_step` / `value` are per single call; `steps` and `warmup` echo the command line.

Extra objects on the same line:
  roofline     the matvec kernel alone (activations quantized before the timed region), timed
               with HIP events on the library's stream over the same rotation; with `fit`: launch time against
               bytes over six weight sizes for this kernel and for a kernel that only reads (fixed_us,
               marginal_GBps), `launch_split`: empty kernels and one-load kernels, and `sustained`: the same kernel
               with the fixed part amortised (2 or 3 weights per launch) or hidden (two streams).
  cpu_baseline candy's literal CPU composition (dequantize, then the naive f32 matmul loops)
               restated in C, single thread, on a bounded sample of the same workload.
  sweep        the other shapes / formats of the batch-1 sweep (GB/s of the matvec kernel).
  decode       random-init 7B Q4_K decode step, tokens/s.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth
MFMA_F16_PEAK_TFLOPS = 2500.0  # MI355X published dense fp16 MFMA rate
MFMA_I8_PEAK_TOPS = 5000.0  # MI355X published dense int8 MFMA rate
ROTATE_BYTES = 640 << 20  # distinct weight bytes cycled through (last-level cache is 256 MB)
# HBM bytes one launch of the Q4_K 4096x11008 matvec moves: written by `bench.py --write-traffic DIR` from the
# two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) whose commands profiles/matvec_q4k_4096x11008.md gives
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "matvec_q4k_4096x11008_traffic.txt")


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def read_traffic():
    """HBM bytes per launch of the headline kernel from the committed counter summary, or None."""
    try:
        kv = dict(line.split(None, 1) for line in open(TRAFFIC_FILE) if line.strip() and not line.startswith("#"))
        return int(kv["traffic_bytes"])
    except (OSError, KeyError, ValueError):
        return None


def write_traffic(prof_dir):
    """Summarise DIR/fetch_counter_collection.csv and DIR/write_counter_collection.csv (rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE over `bench.py ... --calibrate-copy`) into TRAFFIC_FILE.  Each counter is scaled by what it reads for
    the 256 MiB device-to-device copy of the same run."""
    import csv
    copy_kib = 256 * 1024

    def means(path):
        acc = {}
        for r in csv.DictReader(open(path)):
            acc.setdefault(r["Kernel_Name"], []).append(float(r["Counter_Value"]))
        return {k: sum(v) / len(v) for k, v in acc.items()}

    out = {}
    for tag, name in (("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")):
        m = means(os.path.join(prof_dir, f"{tag}_counter_collection.csv"))
        copy = [v for k, v in m.items() if "copyBuffer" in k]
        mv = [(k, v) for k, v in m.items() if "k_matvec1<candy::UnitQ4K, 3, 1, 4>" in k or "k_matvec1<candy::UnitQ4K,3,1,4>" in k]
        if not copy or not mv:
            sys.exit(f"bench.py --write-traffic: no copy or matvec dispatches in the {name} run under {prof_dir}")
        out[tag] = (mv[0][1], copy_kib / copy[0])
    traffic = int(round((out["fetch"][0] * out["fetch"][1] + out["write"][0] * out["write"][1]) * 1024))
    with open(TRAFFIC_FILE, "w") as f:
        f.write("# k_matvec1<UnitQ4K,3,1,4>, Q4_K 4096x11008 batch 1: HBM bytes per launch from rocprofv3 --pmc\n")
        f.write("# (KiB per dispatch, mean over dispatches; factor = 262144 KiB / what the counter reads for a 256 MiB copy)\n")
        f.write(f"fetch_KiB_raw {out['fetch'][0]:.1f}\nfetch_factor {out['fetch'][1]:.4f}\n")
        f.write(f"write_KiB_raw {out['write'][0]:.1f}\nwrite_factor {out['write'][1]:.4f}\n")
        f.write(f"traffic_bytes {traffic}\n")
    print(open(TRAFFIC_FILE).read())


def stream_floor(dev, nbytes):
    """What a kernel that only reads achieves on this device, measured now: GB/s for launches of `nbytes` rotating
    over ROTATE_BYTES, GB/s for one pass over ROTATE_BYTES, and microseconds per launch of an empty kernel."""
    span = ROTATE_BYTES // nbytes * nbytes
    us_small = dev.stream_probe(nbytes, span, 400) / 400 * 1e3
    us_big = dev.stream_probe(span, span, 10) / 10 * 1e3
    us_empty = dev.stream_probe(0, 0, 1000) / 1000 * 1e3
    return nbytes / us_small / 1e3, span / us_big / 1e3, us_empty, us_small


def algorithmic_bytes(fmt, rows, cols, m=1):
    from candy_amd import synth
    return synth.weight_nbytes(fmt, rows, cols) + 4 * m * cols + 4 * m * rows


def make_rotation(dev, fmt, rows, cols, seed):
    """Distinct device copies of one random weight shape, >= ROTATE_BYTES in total."""
    from candy_amd import synth
    nbytes = synth.weight_nbytes(fmt, rows, cols)
    n = max(2, -(-ROTATE_BYTES // nbytes))
    base = synth.random_weight(fmt, rows, cols, seed=seed)
    ws = []
    for i in range(n):
        # cheap distinct contents: rotate the block array (still valid blocks, still random)
        blk = synth.BLOCK_BYTES[fmt]
        ws.append(dev.qtensor(fmt, rows, cols, np.roll(base.reshape(-1, blk), i, axis=0).reshape(-1)))
    return ws, nbytes


def time_matvec(dev, fmt, rows, cols, steps, warmup, quantize_each, seed=1, m=1):
    from candy_amd import synth
    ws, nbytes = make_rotation(dev, fmt, rows, cols, seed)
    x = dev.from_numpy(synth.random_activations(m, cols, seed=seed + 1))
    y = dev.alloc(4 * m * rows)
    dev.qmatmul_sweep(ws, x, m, y, warmup, quantize_each)
    ms = dev.qmatmul_sweep(ws, x, m, y, steps, quantize_each)
    for w in ws:
        w.free()
    return ms / steps, len(ws)


def linear_fit(xs, ys):
    """Least squares y = a + b x."""
    n = len(xs)
    mx, my = sum(xs) / n, sum(ys) / n
    b = sum((x - mx) * (y - my) for x, y in zip(xs, ys)) / sum((x - mx) ** 2 for x in xs)
    return my - b * mx, b


def launch_fit(dev, fmt, cols, launches):
    """Launch time against bytes for the batch-1 kernel and for a kernel that only reads the same bytes, over six
    weight sizes (rows 1024 .. 32768 at `cols` columns, 6 .. 203 MB of Q4_K), every launch on weights not in any
    cache: time = fixed_us + bytes / marginal_GBps."""
    from candy_amd import synth
    pts = []
    for rows in (1024, 2048, 4096, 8192, 16384, 32768):
        nb = synth.weight_nbytes(fmt, rows, cols)
        ms, _ = time_matvec(dev, fmt, rows, cols, launches, max(20, launches // 10), quantize_each=False, seed=rows)
        span = max(2, -(-ROTATE_BYTES // nb)) * nb
        us_read = dev.stream_probe(nb, span, launches) / launches * 1e3
        pts.append({"rows": rows, "weight_bytes": nb, "matvec_us": round(ms * 1e3, 3), "read_only_us": round(us_read, 3)})
        log(f"  fit {rows}x{cols}: {nb / 1e6:.1f} MB, matvec {ms * 1e3:.2f} us, read-only {us_read:.2f} us")
    out = {"points": pts}
    for key, name in (("matvec_us", "matvec"), ("read_only_us", "read_only")):
        a, b = linear_fit([p["weight_bytes"] for p in pts], [p[key] for p in pts])
        worst = max(abs(a + b * p["weight_bytes"] - p[key]) / p[key] for p in pts)
        out[name] = {"fixed_us": round(a, 3), "marginal_GBps": round(1e-3 / b, 1), "max_rel_residual": round(worst, 4)}
    return out


def launch_split(dev, n=2000):
    """Where the fixed part goes: microseconds per launch of empty kernels and of kernels whose wavefronts issue
    exactly one load."""
    names = ("empty_1_wavefront_us", "empty_1024x256_us", "one_load_per_wavefront_warm_us", "one_load_per_wavefront_cold_us")
    return {name: round(dev.launch_probe(kind, n) / n * 1e3, 3) for kind, name in enumerate(names)}


def sustained(dev, fmt, rows, cols, launches):
    """The batch-1 kernel at the headline shape with the fixed part of a launch amortised (2 or 3 independent weights
    sharing x in one launch: the q / k / v mechanism) or hidden (launches alternating over two streams).  Independent
    contractions only - not the headline."""
    from candy_amd import synth
    ws, nbytes = make_rotation(dev, fmt, rows, cols, seed=31)
    x = dev.from_numpy(synth.random_activations(1, cols, seed=32))
    y = dev.alloc(4 * rows * 6)
    out = {"note": "independent contractions (no launch waits for the previous one's result); bytes = weights + x + y "
                   "per contraction; NOT the headline: a single serialized launch is roofline.us_per_launch"}
    per = algorithmic_bytes(fmt, rows, cols)
    for key, group, streams in (("weights_per_launch_2", 2, 1), ("weights_per_launch_3", 3, 1), ("two_streams", 1, 2),
                                ("two_streams_weights_per_launch_3", 3, 2)):
        dev.qmatmul_sustained_sweep(ws, group, streams, x, y, max(20, launches // 10))
        ms = dev.qmatmul_sustained_sweep(ws, group, streams, x, y, launches) / launches
        gb = per * group / (ms * 1e-3) / 1e9
        out[key] = {"us_per_launch": round(ms * 1e3, 3), "us_per_contraction": round(ms * 1e3 / group, 3),
                    "GBps": round(gb, 1), "frac": round(gb / HBM_PEAK_GBPS, 4)}
        log(f"  sustained {key}: {ms * 1e3:.2f} us per launch, {gb:.0f} GB/s ({gb / HBM_PEAK_GBPS:.1%})")
    for w in ws:
        w.free()
    x.free()
    y.free()
    return out


def cpu_baseline(rows, cols, budget_s=12.0):
    """candy's CPU path (dequantize + naive f32 loops), C restatement, one thread."""
    from candy_amd import synth
    from oracle import oracle as o
    fmt = synth.Q4_K
    sample_rows = 512  # a slice of the same weight keeps one call short
    w = synth.random_weight(fmt, sample_rows, cols, seed=77)
    x = synth.random_activations(1, cols, seed=78)
    o.matmul_dequant_f32(fmt, w, sample_rows, cols, x)  # warm
    t0 = time.perf_counter()
    calls = 0
    while time.perf_counter() - t0 < budget_s:
        o.matmul_dequant_f32(fmt, w, sample_rows, cols, x)
        calls += 1
    dt = time.perf_counter() - t0
    per_full = dt / calls * (rows / sample_rows)
    gbps = algorithmic_bytes(fmt, rows, cols) / per_full / 1e9
    return {"value": round(gbps, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{calls} calls of dequantize+naive-f32-matmul on a {sample_rows}x{cols} Q4_K slice "
                      f"({dt:.1f} s), scaled to {rows} rows; host has {os.cpu_count()} logical CPUs",
            "ms_per_step": round(per_full * 1e3, 3)}


def quantized_normal(dev, fmt, rows, cols, seed, std=0.02):
    """Blocks of a [rows, cols] matrix drawn from N(0, std) and quantized by the library's own quantizer on the device."""
    rng = np.random.Generator(np.random.Philox(seed))
    x = rng.standard_normal((rows, cols), dtype=np.float32) * np.float32(std)
    return dev.quantize(fmt, x)


def build_7b(dev, n_layers=32, max_pos=2176, seed=4000):
    """Random-init Llama-7B-shaped decoder: Q4_K linears, Q6_K head, Q8_0 embedding rows; weights drawn from
    N(0, 0.02) and then quantized on the device.  One draw per shape; the layers take it with its blocks rotated
    (distinct contents, same distribution) so that building the model stays a matter of seconds."""
    from candy_amd import hip, synth
    cfg = dict(n_layers=n_layers, d_model=4096, n_heads=32, n_kv_heads=32, head_dim=128, d_ffn=11008, vocab=32000,
               max_pos=max_pos, rms_eps=1e-5, rope_base=10000.0)
    model = hip.Llama(dev, **cfg)
    shapes = [(hip.W_Q, 4096, 4096), (hip.W_K, 4096, 4096), (hip.W_V, 4096, 4096), (hip.W_O, 4096, 4096),
              (hip.W_GATE, 11008, 4096), (hip.W_UP, 11008, 4096), (hip.W_DOWN, 4096, 11008)]
    ones = np.ones(4096, np.float32)
    t0 = time.perf_counter()
    base = {(r, k): quantized_normal(dev, synth.Q4_K, r, k, seed + r + k).reshape(-1, synth.BLOCK_BYTES[synth.Q4_K])
            for r, k in {(r, k) for _, r, k in shapes}}
    shift = 0
    for l in range(n_layers):
        for kind, r, k in shapes:
            shift += 1
            model.set_qweight(kind, l, dev.qtensor(synth.Q4_K, r, k, np.roll(base[(r, k)], 977 * shift, axis=0).reshape(-1)))
        model.set_norm(hip.W_ATTN_NORM, l, ones)
        model.set_norm(hip.W_FFN_NORM, l, ones)
        if l % 8 == 7:
            log(f"  built layer {l + 1}/{n_layers} ({time.perf_counter() - t0:.0f} s)")
    model.set_norm(hip.W_OUT_NORM, -1, ones)
    model.set_qweight(hip.W_HEAD, -1, dev.qtensor(synth.Q6_K, 32000, 4096, quantized_normal(dev, synth.Q6_K, 32000, 4096, seed + 1)))
    model.set_qweight(hip.W_EMBED, -1, dev.qtensor(synth.Q8_0, 32000, 4096, quantized_normal(dev, synth.Q8_0, 32000, 4096, seed + 2)))
    return cfg, model


def build_8b(dev, max_pos, seed=8000):
    """Random-init Llama-3-8B-shaped decoder: GQA 32/8, FFN 14336, vocab 128256; Q4_K attention and
    gate/up, Q6_K down and head, Q8_0 embedding rows."""
    from candy_amd import hip, synth
    cfg = dict(n_layers=32, d_model=4096, n_heads=32, n_kv_heads=8, head_dim=128, d_ffn=14336, vocab=128256,
               max_pos=max_pos, rms_eps=1e-5, rope_base=500000.0)
    model = hip.Llama(dev, **cfg)
    shapes = [(hip.W_Q, 4096, 4096, synth.Q4_K), (hip.W_K, 1024, 4096, synth.Q4_K), (hip.W_V, 1024, 4096, synth.Q4_K),
              (hip.W_O, 4096, 4096, synth.Q4_K), (hip.W_GATE, 14336, 4096, synth.Q4_K),
              (hip.W_UP, 14336, 4096, synth.Q4_K), (hip.W_DOWN, 4096, 14336, synth.Q6_K)]
    ones = np.ones(4096, np.float32)
    t0 = time.perf_counter()
    nbytes = 0
    for l in range(cfg["n_layers"]):
        for kind, r, k, f in shapes:
            seed += 1
            model.set_qweight(kind, l, dev.qtensor(f, r, k, synth.random_weight(f, r, k, seed, synth.unit_scale(f))))
            nbytes += synth.weight_nbytes(f, r, k)
        model.set_norm(hip.W_ATTN_NORM, l, ones)
        model.set_norm(hip.W_FFN_NORM, l, ones)
        if l % 8 == 7:
            log(f"  built layer {l + 1}/32 ({time.perf_counter() - t0:.0f} s)")
    model.set_norm(hip.W_OUT_NORM, -1, ones)
    model.set_qweight(hip.W_HEAD, -1, dev.qtensor(synth.Q6_K, 128256, 4096, synth.random_weight(
        synth.Q6_K, 128256, 4096, seed + 1, synth.unit_scale(synth.Q6_K))))
    model.set_qweight(hip.W_EMBED, -1, dev.qtensor(synth.Q8_0, 128256, 4096, synth.random_weight(
        synth.Q8_0, 128256, 4096, seed + 2, synth.unit_scale(synth.Q8_0))))
    return cfg, model, nbytes + synth.weight_nbytes(synth.Q6_K, 128256, 4096)


def llama3_leg(dev, n_prompt=512, n_decode=128, not_eager=True):
    """Prefill a seeded random prompt in one batched pass, then decode greedily at batch 1."""
    log("building random-init Llama-3-8B shape (Q4_K / Q6_K down+head / Q8_0 embedding) ...")
    cfg, model, weight_bytes = build_8b(dev, max_pos=n_prompt + n_decode + 8)
    prompt = [int(t) for t in np.random.default_rng(4321).integers(0, cfg["vocab"], n_prompt)]
    model.prefill(prompt[:64], 0, want_logits=False)  # warm-up: allocates the prompt buffers' first size
    model.prefill(prompt, 0, want_logits=False)
    dev.synchronize()
    # The chip raises its clocks over the first 100 ms or so of matrix-core load (a 512-row contraction takes 85 us in
    # the first milliseconds and 75 us from then on): the first three passes are timed as they come, then the
    # sustained figure after ten more.
    t0 = time.perf_counter()
    for _ in range(3):
        tok, _ = model.prefill(prompt, 0, want_logits=False)
    dev.synchronize()
    first_s = (time.perf_counter() - t0) / 3
    for _ in range(10):
        model.prefill(prompt, 0, want_logits=False)
    dev.synchronize()
    t0 = time.perf_counter()
    reps = 5
    for _ in range(reps):
        tok, _ = model.prefill(prompt, 0, want_logits=False)
    dev.synchronize()
    pre_s = (time.perf_counter() - t0) / reps
    pos = n_prompt
    # the first decoded token twice: as a replay of the captured graph and as one-by-one launches (same kernels, same
    # cache slot rewritten with the same rows) - they must agree
    first_graph, _ = model.decode(tok, pos, want_logits=False)
    model.set_graph(False)
    first_eager, _ = model.decode(tok, pos, want_logits=False)
    model.set_graph(not_eager)
    for _ in range(4):
        tok, _ = model.decode(tok, pos, want_logits=False)
        pos += 1
    dev.synchronize()
    # greedy generation, the chosen token handed to the next step on the device (candy_hip_llama_generate): one
    # copy of the token list at the end instead of a device round trip per token
    t0 = time.perf_counter()
    toks = model.generate(tok, pos, n_decode - 4)
    dev.synchronize()
    dec_s = (time.perf_counter() - t0) / (n_decode - 4)
    kv_mid = 2 * cfg["n_layers"] * cfg["n_kv_heads"] * (n_prompt + n_decode // 2) * cfg["head_dim"] * 4
    bpt = weight_bytes + kv_mid
    per_layer_macs = (2 * 4096 * 4096 + 2 * 1024 * 4096 + 3 * 14336 * 4096)
    lin_flops = 2.0 * n_prompt * per_layer_macs * cfg["n_layers"]
    model.free()
    return {"prefill_tokens": n_prompt, "prefill_ms": round(pre_s * 1e3, 2), "prefill_tok_s": round(n_prompt / pre_s, 1),
            "prefill_ms_first_passes": round(first_s * 1e3, 2),
            "prefill_linear_TFLOPs": round(lin_flops / pre_s / 1e12, 1),
            "decode_tokens": n_decode - 4, "decode_ms_per_token": round(dec_s * 1e3, 4), "decode_tok_s": round(1 / dec_s, 2),
            "decode_bytes_per_token": bpt, "decode_hbm_frac": round(bpt / dec_s / 1e9 / HBM_PEAK_GBPS, 4),
            "tokens": toks[:8], "first_token": first_graph, "first_token_graph_equals_eager": first_graph == first_eager}


def prefill_kv(dev, model, cfg, n_pos, seed=9):
    """KV cache positions [0, n_pos) <- N(0,1), in the cache's element type (f32, or fp16 after set_kv_f16)."""
    from candy_amd import hip
    kptr, vptr, nbytes = model.kv_cache()
    rng = np.random.Generator(np.random.Philox(seed))
    per_head = cfg["max_pos"] * cfg["head_dim"]
    elem = nbytes // (cfg["n_layers"] * cfg["n_kv_heads"] * per_head)
    dt = {4: np.float32, 2: np.float16}[elem]
    chunk = np.empty((cfg["n_kv_heads"], n_pos, cfg["head_dim"]), np.float32)
    for base in (kptr, vptr):
        for l in range(cfg["n_layers"]):
            rng.standard_normal(chunk.shape, dtype=np.float32, out=chunk)
            rows = chunk.astype(dt)
            for h in range(cfg["n_kv_heads"]):
                off = ((l * cfg["n_kv_heads"] + h) * per_head) * elem
                hip._check(hip.lib().candy_hip_h2d(dev.handle, base + off, rows[h].ctypes.data, rows[h].nbytes))


def decode_leg(dev, steps, warmup, fp16_kv=True):
    from candy_amd import synth
    log("building random-init 7B (N(0, 0.02) quantized to Q4_K, Q6_K head) ...")
    n_pos = 2048
    cfg, model = build_7b(dev, max_pos=n_pos + steps + warmup + 8)
    layer_bytes = 4 * synth.weight_nbytes(synth.Q4_K, 4096, 4096) + 3 * synth.weight_nbytes(synth.Q4_K, 11008, 4096)
    weight_bytes = cfg["n_layers"] * layer_bytes + synth.weight_nbytes(synth.Q6_K, 32000, 4096)

    def run(kv_elem_bytes):
        prefill_kv(dev, model, cfg, n_pos)
        tok = int(np.random.default_rng(1234).integers(0, cfg["vocab"], 128)[-1])
        pos = n_pos
        for _ in range(warmup):
            tok, _ = model.decode(tok, pos, want_logits=False)
            pos += 1
        dev.synchronize()
        # the timed region: `steps` greedy steps, each step's token handed to the next on the device
        # (candy_hip_llama_generate), the token list copied out once at the end
        t0 = time.perf_counter()
        toks = model.generate(tok, pos, steps)
        dev.synchronize()
        dt = time.perf_counter() - t0
        # beside it: the same steps with the host fetching every token (candy_hip_llama_decode in a loop)
        tok2, pos2 = toks[-1], pos + steps
        t1 = time.perf_counter()
        for _ in range(min(steps, 16)):
            tok2, _ = model.decode(tok2, pos2 - 1, want_logits=False)
        dev.synchronize()
        fetched = (time.perf_counter() - t1) / min(steps, 16)
        kv_bytes = 2 * cfg["n_layers"] * cfg["n_kv_heads"] * n_pos * cfg["head_dim"] * kv_elem_bytes
        bpt = weight_bytes + kv_bytes
        ms = dt / steps * 1e3
        return {"tok_s": round(steps / dt, 2), "ms_per_token": round(ms, 4), "steps": steps, "kv_positions": n_pos,
                "bytes_per_token": bpt, "hbm_GBps": round(bpt / (ms * 1e-3) / 1e9, 1),
                "hbm_frac": round(bpt / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4), "tokens": toks[:8],
                "tok_s_token_fetched_every_step": round(1 / fetched, 2)}

    out = run(4)  # candy's cache is f32: this is the figure quoted
    # the optional half-size cache, beside it (k and v rounded to fp16 on entry; not what the reference computes)
    if fp16_kv:
        model.set_kv_f16(True)
        half = run(2)
        out["fp16_kv_cache"] = {k: half[k] for k in ("tok_s", "ms_per_token", "bytes_per_token", "hbm_GBps", "hbm_frac")}
    model.free()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-fit", action="store_true", help="skip the launch-time fit, launch split and sustained figures")
    ap.add_argument("--fit-only", action="store_true", help="stop after the headline, fit, launch split and sustained figures")
    ap.add_argument("--no-sweep", action="store_true", help="skip the other shapes of the batch-1 sweep")
    ap.add_argument("--no-decode", action="store_true", help="skip the 7B decode leg")
    ap.add_argument("--no-prefill", action="store_true", help="skip the batched-prefill (MFMA) leg")
    ap.add_argument("--prefill-steps", type=int, default=1000, help="timed calls per batch size of the prefill leg")
    ap.add_argument("--prefill-warmup-ms", type=float, default=150.0,
                    help="untimed calls in front of them, as milliseconds of work (the matrix-core kernels run 10-20 %% "
                         "slower until the chip has raised its clocks); a counter run wants few dispatches: 0")
    ap.add_argument("--no-llama3", action="store_true", help="skip the Llama-3-8B-shaped prefill + decode leg")
    ap.add_argument("--decode-steps", type=int, default=32)
    ap.add_argument("--eager", action="store_true",
                    help="decoders launch their kernels one by one instead of replaying a captured HIP graph (for "
                         "profiler runs: each launch is then a dispatch the tool sees on its own)")
    ap.add_argument("--no-fp16-kv", action="store_true", help="skip the decode leg's second figure (fp16 KV cache)")
    ap.add_argument("--option", action="append", default=[], metavar="KEY=VALUE",
                    help="set a library option (candy_hip_set_option) before anything runs; comparison runs only")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one 256 MiB device-to-device copy (a kernel of known traffic for counter runs)")
    ap.add_argument("--write-traffic", metavar="DIR",
                    help="no benchmark: summarise the FETCH_SIZE / WRITE_SIZE runs under DIR into " + TRAFFIC_FILE)
    args = ap.parse_args()
    if args.write_traffic:
        write_traffic(args.write_traffic)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on ONE MI355X; --gpus must be 1 (no collectives, no sharding)")

    from candy_amd import hip, synth
    dev = hip.Device(0)
    log("device:", dev.name)
    for kv in args.option:
        key, _, val = kv.partition("=")
        dev.set_option(key, int(val))
    if args.eager:
        dev.set_option("llama.graph", 0)
    fmt, rows, cols = synth.Q4_K, 4096, 11008
    alg = algorithmic_bytes(fmt, rows, cols)
    if args.calibrate_copy:
        a, b = dev.alloc(256 << 20), dev.alloc(256 << 20)
        a.zero()
        hip._check(hip.lib().candy_hip_d2d(dev.handle, b.ptr, a.ptr, 256 << 20))
        dev.synchronize()
        a.free()
        b.free()

    # headline: whole f32-in -> f32-out path.  Every step is inner_reps calls back to back (>= 1000 timed calls whatever
    # --steps is: twenty calls are 0.2 ms, one short sample); figures are per single call.
    inner = max(1, -(-1000 // max(args.steps, 1)))
    n_timed, n_warm = args.steps * inner, max(args.warmup * inner, 50)
    ms_step, n_copies = time_matvec(dev, fmt, rows, cols, n_timed, n_warm, quantize_each=True)
    value = alg / (ms_step * 1e-3) / 1e9
    # dominant kernel alone
    ms_kernel, _ = time_matvec(dev, fmt, rows, cols, n_timed, n_warm, quantize_each=False)
    achieved = alg / (ms_kernel * 1e-3) / 1e9
    log(f"Q4_K {rows}x{cols}: path {ms_step * 1e3:.2f} us/step = {value:.0f} GB/s; "
        f"matvec kernel {ms_kernel * 1e3:.2f} us = {achieved:.0f} GB/s ({achieved / HBM_PEAK_GBPS:.1%} of 8 TB/s)")
    # the same bytes through a kernel that only reads them, and an empty kernel: the floor under any launch
    floor_small, floor_big, us_empty, us_floor = stream_floor(dev, synth.weight_nbytes(fmt, rows, cols))
    log(f"read-only stream: {floor_small:.0f} GB/s at {synth.weight_nbytes(fmt, rows, cols)} B per launch ({us_floor:.2f} us), "
        f"{floor_big:.0f} GB/s over {ROTATE_BYTES >> 20} MiB in one launch; empty kernel {us_empty:.2f} us per launch")

    out = {
        "metric": "Q4_K matvec GB/s (batch 1, 4096x11008, f32 in -> f32 out)",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "i8", "data": "synthetic",
        "config": {"workload": "configs[1]: Q4_K 4096x11008 (N x K) batch-1 matvec, activation quantized to Q8_0 "
                               "on device each step", "weight_bytes": synth.weight_nbytes(fmt, rows, cols),
                   "algorithmic_bytes_per_step": alg, "distinct_weight_copies": n_copies,
                   "inner_reps": inner, "timed_calls": n_timed, "device": dev.name,
                   "decode_model": "random-init 7B: one N(0, 0.02) draw per weight shape quantized on the device by "
                                   "candy_hip_quantize (Q4_K / Q6_K quantizers restate ggml's published reference "
                                   "quantizers; parity unpinned against ggml itself), each layer taking the draw "
                                   "with its blocks rotated"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": read_traffic(),
                     "kernel": "k_matvec1<UnitQ4K,3,1,4>", "us_per_launch": round(ms_kernel * 1e3, 3),
                     "achievable_GBps_25MB": round(floor_small, 1), "achievable_GBps_stream": round(floor_big, 1),
                     "empty_launch_us": round(us_empty, 3), "frac_of_achievable": round(achieved / floor_small, 4)},
    }
    if not args.no_fit:
        log("launch time against bytes (six sizes), launch split, sustained figures ...")
        out["roofline"]["fit"] = launch_fit(dev, fmt, cols, 400)
        out["roofline"]["launch_split"] = launch_split(dev)
        out["roofline"]["sustained"] = sustained(dev, fmt, rows, cols, 1000)
    if args.fit_only:
        dev.close()
        print(json.dumps(out))
        return

    if not args.no_sweep:
        sweep = []
        s_steps, s_warm = max(200, args.steps // 4), max(20, args.warmup // 4)
        for f, name in ((synth.Q4_K, "q4_k"), (synth.Q8_0, "q8_0")):
            for r, k in ((4096, 4096), (11008, 4096), (4096, 11008), (32000, 4096)):
                ms, _ = time_matvec(dev, f, r, k, s_steps, s_warm, quantize_each=False, seed=r + k)
                gb = algorithmic_bytes(f, r, k) / (ms * 1e-3) / 1e9
                sweep.append({"fmt": name, "rows": r, "cols": k, "us": round(ms * 1e3, 3), "GBps": round(gb, 1),
                              "frac": round(gb / HBM_PEAK_GBPS, 4)})
                log(f"  {name} {r}x{k}: {ms * 1e3:.2f} us, {gb:.0f} GB/s")
        for f, name, r, k in ((synth.Q6_K, "q6_k", 32000, 4096), (synth.Q4_0, "q4_0", 4096, 4096)):
            ms, _ = time_matvec(dev, f, r, k, s_steps, s_warm, quantize_each=False, seed=r + k + f)
            gb = algorithmic_bytes(f, r, k) / (ms * 1e-3) / 1e9
            sweep.append({"fmt": name, "rows": r, "cols": k, "us": round(ms * 1e3, 3), "GBps": round(gb, 1),
                          "frac": round(gb / HBM_PEAK_GBPS, 4)})
            log(f"  {name} {r}x{k}: {ms * 1e3:.2f} us, {gb:.0f} GB/s")
        # the reference's other formats (same batch-1 kernel template, no span staging, no fused decode kernels)
        for f in (synth.Q4_1, synth.Q5_0, synth.Q5_1, synth.Q2_K, synth.Q3_K, synth.Q5_K):
            r, k, name = 4096, 11008, synth.FORMAT_NAMES[f]
            ms, _ = time_matvec(dev, f, r, k, s_steps, s_warm, quantize_each=False, seed=r + k + f)
            gb = algorithmic_bytes(f, r, k) / (ms * 1e-3) / 1e9
            sweep.append({"fmt": name, "rows": r, "cols": k, "us": round(ms * 1e3, 3), "GBps": round(gb, 1),
                          "frac": round(gb / HBM_PEAK_GBPS, 4)})
            log(f"  {name} {r}x{k}: {ms * 1e3:.2f} us, {gb:.0f} GB/s")
        out["sweep"] = sweep
        # small batches (mul_mat_vec_q serves 1..8 rows in the reference): f32 in -> f32 out, quantization included
        small = []
        for f, r, k in ((synth.Q4_K, 4096, 11008), (synth.Q4_K, 11008, 4096), (synth.Q6_K, 32000, 4096)):
            for m in (2, 4, 8, 15, 16, 32):
                ms, _ = time_matvec(dev, f, r, k, s_steps, s_warm, quantize_each=True, seed=r + k + f + m, m=m)
                small.append({"fmt": synth.FORMAT_NAMES[f], "rows": r, "cols": k, "m": m, "us": round(ms * 1e3, 2),
                              "GBps": round(algorithmic_bytes(f, r, k, m) / (ms * 1e-3) / 1e9, 1)})
                log(f"  {synth.FORMAT_NAMES[f]} {r}x{k} m={m}: {ms * 1e3:.2f} us")
        out["small_batch"] = small
        # the reference's other matvec: f32 activations, no activation quantizer (dequantize_mul_mat_vec)
        dm = []
        for f, r, k in ((synth.Q4_K, 4096, 11008), (synth.Q4_K, 11008, 4096), (synth.Q6_K, 32000, 4096)):
            ws, nbytes = make_rotation(dev, f, r, k, seed=r + k + 3)
            x = dev.from_numpy(synth.random_activations(1, k, seed=5))
            y = dev.alloc(4 * r)
            for timed in (False, True):
                dev.synchronize()
                dev.timer_start()
                for i in range(s_steps):
                    hip._check(hip.lib().candy_hip_dmmv(dev.handle, ws[i % len(ws)].handle, x.ptr, y.ptr))
                ms = dev.timer_stop() / s_steps
            for w in ws:
                w.free()
            dm.append({"fmt": synth.FORMAT_NAMES[f], "rows": r, "cols": k, "us": round(ms * 1e3, 2),
                       "GBps": round(algorithmic_bytes(f, r, k) / (ms * 1e-3) / 1e9, 1)})
            log(f"  dmmv {synth.FORMAT_NAMES[f]} {r}x{k}: {ms * 1e3:.2f} us")
        out["dmmv"] = dm

    if not args.no_sweep:
        # weight quantizers from f32 (load-time): 4096x11008, one launch each
        wq = []
        r, k = 4096, 11008
        xw = dev.from_numpy((np.random.default_rng(77).standard_normal((r, k)) * 0.02).astype(np.float32))
        for f in (synth.Q4_0, synth.Q8_0, synth.Q4_K, synth.Q6_K):
            dst = dev.alloc(synth.weight_nbytes(f, r, k))
            for rep in range(2):
                dev.synchronize()
                t0 = time.perf_counter()
                hip._check(hip.lib().candy_hip_quantize(dev.handle, f, xw.ptr, r, k, dst.ptr))
                dev.synchronize()
                dt = time.perf_counter() - t0
            wq.append({"op": "quantize", "fmt": synth.FORMAT_NAMES[f], "rows": r, "cols": k, "ms": round(dt * 1e3, 3),
                       "Gvalues_s": round(r * k / dt / 1e9, 1)})
            log(f"  quantize {synth.FORMAT_NAMES[f]} {r}x{k}: {dt * 1e3:.2f} ms")
            dst.free()
        xw.free()
        out["weight_quantizers"] = wq

    if not args.no_sweep:
        # the two conversions, both HBM-bound: dequantize writes 4 B per weight, quantize reads 4 B per value.  Inputs AND
        # outputs rotate over more than ROTATE_BYTES each, so neither side is served from the 256 MB last-level cache.
        conv = []
        for f, name in ((synth.Q4_K, "q4_k"), (synth.Q6_K, "q6_k"), (synth.Q8_0, "q8_0"), (synth.Q4_0, "q4_0")):
            r, k = 4096, 11008
            nb = synth.weight_nbytes(f, r, k)
            ws, _ = make_rotation(dev, f, r, k, seed=500 + f)
            n_out = -(-ROTATE_BYTES // (4 * r * k))
            outb = dev.alloc(4 * r * k * n_out)
            dev.dequantize_sweep(ws, outb, 10, n_out)
            ms = dev.dequantize_sweep(ws, outb, 60, n_out) / 60
            byts = nb + 4 * r * k
            conv.append({"op": "dequantize", "fmt": name, "rows": r, "cols": k, "us": round(ms * 1e3, 2),
                         "GBps": round(byts / (ms * 1e-3) / 1e9, 1), "frac": round(byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                         "rotation": f"{len(ws)} inputs, {n_out} outputs ({(nb * len(ws) + 4 * r * k * n_out) >> 20} MiB)"})
            log(f"  dequantize {name} {r}x{k}: {ms * 1e3:.1f} us, {conv[-1]['GBps']} GB/s")
            for w in ws:
                w.free()
            outb.free()
        for r, k in ((1, 4096), (512, 4096)):
            in_bytes, out_bytes = 4 * r * k, r * k // 32 * 34
            copies = max(1, min(4096, -(-ROTATE_BYTES // in_bytes)))
            n_out = max(1, min(4096, -(-ROTATE_BYTES // out_bytes)))
            x = dev.alloc(in_bytes * copies)
            x.zero()
            one = synth.random_activations(r, k, seed=9)
            for c in range(min(copies, 64)):  # N(0, 1) in the first copies, zeros in the rest (the time is the same)
                hip._check(hip.lib().candy_hip_h2d(dev.handle, x.ptr + c * in_bytes, one.ctypes.data, in_bytes))
            outb = dev.alloc(out_bytes * n_out + 64)
            dev.quantize_sweep(x, r * k, copies, r, k, outb, 20, n_out)
            ms = dev.quantize_sweep(x, r * k, copies, r, k, outb, 400, n_out) / 400
            byts = in_bytes + out_bytes
            label = "HBM" if in_bytes * copies >= ROTATE_BYTES else "cache-resident (launch-bound: the rotation is %d MiB)" % ((in_bytes * copies) >> 20)
            conv.append({"op": "quantize_q8_0", "rows": r, "cols": k, "us": round(ms * 1e3, 2),
                         "GBps": round(byts / (ms * 1e-3) / 1e9, 1), "frac": round(byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                         "memory": label})
            log(f"  quantize_q8_0 {r}x{k}: {ms * 1e3:.2f} us, {conv[-1]['GBps']} GB/s ({label})")
            x.free()
            outb.free()
        out["conversions"] = conv

    if not args.no_prefill:
        # batched prefill: Q4_K 14336x4096 x f32 [M, 4096], f32 in -> f32 out (activation quantization included).
        # m <= 16 is one pass over the weights on the int8 matrix cores (k_mmv_q4k), 16 < m < 33 the int8 tile kernel
        # (both exact integer dots; peak 5.0 POP/s), m >= 33 fp16 tiles
        # (operands rounded to fp16, 3e-4 per matmul; peak 2.5 PFLOP/s).  roofline_us = the larger of the bytes at 8 TB/s and the contraction at that peak.
        pre = []
        r, k = 14336, 4096
        big_min = dev.get_option("mmq.f16_api_min_m")
        for m in (16, 128, 512):
            # warm-up of about 150 ms: the matrix-core kernels run 10 % slower until the chip has raised its clocks
            warm = max(5, int({16: 2000, 128: 4000, 512: 2000}[m] * args.prefill_warmup_ms / 150.0))
            ms, _ = time_matvec(dev, synth.Q4_K, r, k, args.prefill_steps, warm, quantize_each=True, seed=m, m=m)
            flops = 2.0 * m * r * k
            byts = algorithmic_bytes(synth.Q4_K, r, k, m)
            int8 = m < big_min
            peak = MFMA_I8_PEAK_TOPS if int8 else MFMA_F16_PEAK_TFLOPS
            roof_us = max(byts / (HBM_PEAK_GBPS * 1e9), flops / (peak * 1e12)) * 1e6
            pre.append({"m": m, "kernel": "k_mmv_q4k<1,2,2,8> (int8 MFMA, one pass)" if m <= 16 else
                        ("k_mmq_i8<TileQ4K,%d,1,1> (int8 MFMA)" % (1 if m <= 32 else 4)) if int8 else ("k_mmq_f16_pc<BigQ4K,112,%d> (fp16 MFMA, 112x%d tiles)" % ((128, 128) if m <= 128 else (256, 256))),
                        "us": round(ms * 1e3, 2), "TFLOPs": round(flops / (ms * 1e-3) / 1e12, 1),
                        "mfma_peak_TFLOPs": peak, "mfma_frac": round(flops / (ms * 1e-3) / 1e12 / peak, 4),
                        "GBps": round(byts / (ms * 1e-3) / 1e9, 1), "hbm_frac": round(byts / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                        "roofline_us": round(roof_us, 2), "roofline_frac": round(roof_us / (ms * 1e3), 4)})
            log(f"  prefill q4_k {r}x{k} M={m}: {ms * 1e3:.1f} us, {pre[-1]['TFLOPs']} TFLOP/s, {pre[-1]['GBps']} GB/s, "
                f"{pre[-1]['roofline_frac']:.1%} of its roofline")
        out["prefill"] = pre

    if not args.no_decode:
        out["decode"] = decode_leg(dev, args.decode_steps, 4, fp16_kv=not args.no_fp16_kv)
        log("decode:", out["decode"])

    if not args.no_llama3:
        out["llama3_8b"] = llama3_leg(dev, not_eager=not args.eager)
        log("llama3-8b shape:", out["llama3_8b"])

    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(rows, cols)
        log("cpu baseline:", out["cpu_baseline"])
    else:
        out["cpu_baseline"] = None

    dev.close()
    print(json.dumps(out))


if __name__ == "__main__":
    main()
