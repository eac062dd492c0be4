"""CPU composition of one Llama-style decode step from the oracle's ops.

TEST INFRASTRUCTURE ONLY (see oracle/candy_oracle.c). candy holds no model code, so this
is the sequence of candy CPU kernels a candy Llama block would run, with the quantized
Linear (oracle.qmatmul) in place of MatMul:
  RMSNorm (reduce.go:3071-3092) -> q/k/v -> Rope (reduce.go:3987-4006) -> append to the f32 KV
  cache -> MatMul/FastSoftmax/MatMul attention -> o -> Add -> RMSNorm -> gate/up -> Silu*Mul
  (unary.go:3353-3366) -> down -> Add; final RMSNorm -> head -> FastArgmax (reduce.go:846-862).
"""
from __future__ import annotations

import math

import numpy as np

from . import oracle as o


def rope_tables(max_pos: int, head_dim: int, base: float):
    """cos/sin [max_pos, head_dim/2]: angle(p, i) = p * base^(-2i/d) in float64, stored as f32."""
    i = np.arange(head_dim // 2, dtype=np.float64)
    inv = np.power(np.float64(base), -2.0 * i / head_dim)
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * inv[None, :]
    return np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)


class LlamaRef:
    def __init__(self, cfg: dict, weights: dict, f32_activations: bool = False, kv_f16: bool = False,
                 block_order: int = 0, fp16_operands: bool = False):
        """weights: {(kind, layer): (fmt, blocks) | f32 array}; kinds as in candy_hip.h.
        f32_activations: every Linear is dequantize + f32 matmul (candy's literal CPU composition, conv.go:373-389)
        instead of the Q8_0-activation vec-dot: the same model without the activation quantizer, against which the
        size of that quantizer's noise can be measured.
        kv_f16: k (after Rope) and v are rounded to fp16 (nearest even) as they enter the cache; attention reads the
        rounded values as f32.  candy's cache is f32: this models the device's optional half-size cache, nothing else.
        block_order: every Linear adds the blocks of a row in another order (oracle.set_block_order: 1 descending,
        2 even then odd, 3 second half first): further correct evaluations of the same model, for measuring how far
        two such evaluations drift apart.
        fp16_operands: every Linear contracts fp16(dequantized weight) with fp16(d * q of the Q8_0 activations) and
        accumulates in f32: the arithmetic of a tile kernel that folds the scales into fp16 operands, for measuring
        what that rounding costs end to end."""
        self.c = cfg
        self.w = weights
        self.f32_activations = f32_activations
        self.kv_f16 = kv_f16
        self.block_order = block_order
        self.fp16_operands = fp16_operands
        self._w16 = {}
        c = cfg
        self.k_cache = np.zeros((c["n_layers"], c["n_kv_heads"], c["max_pos"], c["head_dim"]), np.float32)
        self.v_cache = np.zeros_like(self.k_cache)
        self.cos, self.sin = rope_tables(c["max_pos"], c["head_dim"], c["rope_base"])

    def _lin_rows(self, kind, layer, x, rows, cols):
        """[m, cols] -> [m, rows]; every row is contracted on its own, so m rows equal m calls with one row."""
        fmt, blocks = self.w[(kind, layer)]
        x = np.asarray(x, np.float32).reshape(-1, cols)
        if self.f32_activations:
            return o.matmul_dequant_f32(fmt, blocks, rows, cols, x)
        if self.fp16_operands:
            key = (kind, layer)
            if key not in self._w16:
                self._w16[key] = o.dequantize(fmt, blocks).reshape(rows, cols).astype(np.float16).astype(np.float32)
            xq = o.dequantize(o.Q8_0, o.quantize_q8_0(x)).reshape(-1, cols)  # d * q, exact in f32
            return xq.astype(np.float16).astype(np.float32) @ self._w16[key].T
        o.set_block_order(self.block_order)
        try:
            return o.qmatmul(fmt, blocks, rows, cols, x)
        finally:
            o.set_block_order(0)

    def _lin(self, kind, layer, x, rows, cols):
        return self._lin_rows(kind, layer, x, rows, cols).reshape(-1)

    def embed(self, token: int) -> np.ndarray:
        fmt, blocks = self.w[("embed", -1)]
        rb = o.block_bytes(fmt) * (self.c["d_model"] // o.block_elems(fmt))
        return o.dequantize(fmt, blocks[token * rb:(token + 1) * rb])

    def step(self, h: np.ndarray, pos: int, trace: list | None = None):
        """trace (optional): receives, per layer, the hidden state in front of the layer and the one between its
        attention and feed-forward halves, then the one behind the last layer (2 * n_layers + 1 arrays)."""
        c = self.c
        d, hd, nh, nkv, ffn = c["d_model"], c["head_dim"], c["n_heads"], c["n_kv_heads"], c["d_ffn"]
        h = np.ascontiguousarray(h, np.float32).copy()
        for l in range(c["n_layers"]):
            if trace is not None:
                trace.append(h.copy())
            xn = o.fast_rms_norm(h, d, c["rms_eps"], self.w[("attn_norm", l)])
            q = self._lin("q", l, xn, nh * hd, d)
            k = self._lin("k", l, xn, nkv * hd, d)
            v = self._lin("v", l, xn, nkv * hd, d)
            q = o.rope(q, self.cos[pos], self.sin[pos], nh, hd, hd)
            k = o.rope(k, self.cos[pos], self.sin[pos], nkv, hd, hd)
            if self.kv_f16:
                k, v = k.astype(np.float16).astype(np.float32), v.astype(np.float16).astype(np.float32)
            self.k_cache[l, :, pos, :] = k.reshape(nkv, hd)
            self.v_cache[l, :, pos, :] = v.reshape(nkv, hd)
            att = o.attention_decode(q, self.k_cache[l], self.v_cache[l], nh, nkv, hd, pos + 1,
                                     c["max_pos"] * hd, 1.0 / math.sqrt(hd))
            h = o.add(h, self._lin("o", l, att, d, nh * hd))
            if trace is not None:
                trace.append(h.copy())
            xn = o.fast_rms_norm(h, d, c["rms_eps"], self.w[("ffn_norm", l)])
            g = self._lin("gate", l, xn, ffn, d)
            u = self._lin("up", l, xn, ffn, d)
            act = o.mul(o.silu(g), u)
            h = o.add(h, self._lin("down", l, act, d, ffn))
        if trace is not None:
            trace.append(h.copy())
        xn = o.fast_rms_norm(h, d, c["rms_eps"], self.w[("out_norm", -1)])
        logits = self._lin("head", -1, xn, c["vocab"], d)
        return int(o.fast_argmax(logits, c["vocab"])[0]), logits, h

    def prefill(self, tokens, pos0: int = 0):
        """The step above for tokens at positions pos0, pos0 + 1, ... with every Linear, norm and SiLU*Mul applied to
        all rows at once (each row is treated on its own by those ops, so the result is that of token-by-token
        steps); Rope and attention run token by token over the growing cache.  Returns the last token's
        (greedy next token, logits, hidden state)."""
        c = self.c
        d, hd, nh, nkv, ffn = c["d_model"], c["head_dim"], c["n_heads"], c["n_kv_heads"], c["d_ffn"]
        n = len(tokens)
        h = np.stack([self.embed(int(t)) for t in tokens]).astype(np.float32)
        for l in range(c["n_layers"]):
            xn = o.fast_rms_norm(h, d, c["rms_eps"], self.w[("attn_norm", l)]).reshape(n, d)
            q = self._lin_rows("q", l, xn, nh * hd, d)
            k = self._lin_rows("k", l, xn, nkv * hd, d)
            v = self._lin_rows("v", l, xn, nkv * hd, d)
            att = np.empty((n, nh * hd), np.float32)
            for i in range(n):
                pos = pos0 + i
                qi = o.rope(q[i], self.cos[pos], self.sin[pos], nh, hd, hd)
                ki = o.rope(k[i], self.cos[pos], self.sin[pos], nkv, hd, hd)
                vi = v[i]
                if self.kv_f16:
                    ki, vi = ki.astype(np.float16).astype(np.float32), vi.astype(np.float16).astype(np.float32)
                self.k_cache[l, :, pos, :] = ki.reshape(nkv, hd)
                self.v_cache[l, :, pos, :] = vi.reshape(nkv, hd)
                att[i] = o.attention_decode(qi, self.k_cache[l], self.v_cache[l], nh, nkv, hd, pos + 1,
                                            c["max_pos"] * hd, 1.0 / math.sqrt(hd))
            h = o.add(h, self._lin_rows("o", l, att, d, nh * hd)).reshape(n, d)
            xn = o.fast_rms_norm(h, d, c["rms_eps"], self.w[("ffn_norm", l)]).reshape(n, d)
            g = self._lin_rows("gate", l, xn, ffn, d)
            u = self._lin_rows("up", l, xn, ffn, d)
            act = o.mul(o.silu(g), u).reshape(n, ffn)
            h = o.add(h, self._lin_rows("down", l, act, d, ffn)).reshape(n, d)
        last = h[n - 1]
        xn = o.fast_rms_norm(last, d, c["rms_eps"], self.w[("out_norm", -1)])
        logits = self._lin("head", -1, xn, c["vocab"], d)
        return int(o.fast_argmax(logits, c["vocab"])[0]), logits, last
