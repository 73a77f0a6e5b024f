"""The weight pass of one decode step of a 7B-class model as a list for trn_kquant_gemv_batch: per layer q, k, v, o
(Q4_K 4096x4096), gate, up (Q4_K 11008x4096), down (Q6_K 4096x11008), then the Q6_K 32000x4096 head.  The benchmark and
the parity tests build their lists here, so what is timed is what is checked.

Four ways of wiring the same matrices (`flow`):
  "fresh_x"  a given vector x_l per layer feeds q, k, v, gate, up; o reads the RMS-normalised output of q, down that
             of gate, the head that of the last down.  Activation buffers are shared by all layers, as a decoder's
             are: a layer's q may only be written once the previous layer's o has read it.
  "fresh_x_own_buffers"  the same data flow with activation buffers of its own for every layer: nothing but o <- q and
             down <- gate inside a layer (and head <- the last down) orders the entries, so independent entries of
             neighbouring layers fill the launches.  Same results as "fresh_x", bit for bit.
  "strict"   the serial data flow of a decoder: q, k, v <- h; o <- q; gate, up <- o; down <- gate; h <- down,
             every input RMS-normalised (129 dependent steps).
  "folded"   the decoder layer with its element-wise steps folded into the entries: q, k, v <- rmsnorm(h) * g1;
             h1 = h + o(q); gate, up <- rmsnorm(h1) * g2; h = h1 + down(silu(gate) * up); head <- rmsnorm(h) * g1.
"""
from __future__ import annotations

import numpy as np

from .driver import CudaContext, GpuBuffer
from .kernels import GemvBatch

SB = {"q4k": 144, "q5k": 176, "q6k": 210}
LAYER_MATS = [("q", "q4k", 4096, 4096), ("k", "q4k", 4096, 4096), ("v", "q4k", 4096, 4096), ("o", "q4k", 4096, 4096),
              ("gate", "q4k", 11008, 4096), ("up", "q4k", 11008, 4096), ("down", "q6k", 4096, 11008)]
HEAD = ("head", "q6k", 32000, 4096)
ACT = (("q", 4096), ("k", 4096), ("v", 4096), ("o", 4096), ("gate", 11008), ("up", 11008), ("down", 4096))


def alg_bytes(fmt: str, n: int, k: int) -> int:
    """weights once + x once + y once"""
    return n * (k // 256) * SB[fmt] + 4 * k + 4 * n


class DecodePass:
    """weights: list (one per layer) of {name: GpuBuffer}; head_w: GpuBuffer; xs: per-layer input vectors (4096 f32)
    for flow "fresh_x" (xs[0] is h0 of the other flows)."""

    def __init__(self, ctx: CudaContext, weights, head_w, xs):
        self.ctx, self.weights, self.head_w, self.xs = ctx, weights, head_w, xs
        self.layers = len(weights)
        self.act = {nm: GpuBuffer(ctx, n, np.float32) for nm, n in ACT}
        self.logits = GpuBuffer(ctx, HEAD[2], np.float32)
        self.res = None
        self.gammas = None
        self.act_of_layer = None

    def entry_names(self):
        return [name for _ in range(self.layers) for name, _, _, _ in LAYER_MATS] + ["head"]

    def entry_bytes(self):
        return [alg_bytes(f, n, k) for _ in range(self.layers) for _, f, n, k in LAYER_MATS] + [alg_bytes(*HEAD[1:])]

    def weight_bytes(self):
        return self.layers * sum(n * (k // 256) * SB[f] for _, f, n, k in LAYER_MATS) + HEAD[2] * (HEAD[3] // 256) * SB[HEAD[1]]

    def build(self, flow: str) -> GemvBatch:
        NORM = GemvBatch.NORM_INPUT
        act, b = self.act, GemvBatch()
        if flow in ("fresh_x", "strict"):
            strict = flow == "strict"
            h = self.xs[0]
            for layer in range(self.layers):
                for name, fmt, n, k in LAYER_MATS:
                    if strict:
                        src = {"q": None, "k": None, "v": None, "o": "q", "gate": "o", "up": "o", "down": "gate"}[name]
                        x, flags = (h if src is None else act[src]), NORM
                    else:
                        src = {"o": "q", "down": "gate"}.get(name)
                        x, flags = (self.xs[layer], 0) if src is None else (act[src], NORM)
                    b.add(fmt, k, n, act[name], self.weights[layer][name], x, flags)
                h = act["down"]
            b.add(HEAD[1], HEAD[3], HEAD[2], self.logits, self.head_w, act["down"], NORM)
            return b
        if flow == "fresh_x_own_buffers":
            if self.act_of_layer is None:
                self.act_of_layer = [{nm: GpuBuffer(self.ctx, n, np.float32) for nm, n in ACT} for _ in range(self.layers)]
            for layer in range(self.layers):
                own = self.act_of_layer[layer]
                for name, fmt, n, k in LAYER_MATS:
                    src = {"o": "q", "down": "gate"}.get(name)
                    x, flags = (self.xs[layer], 0) if src is None else (own[src], NORM)
                    b.add(fmt, k, n, own[name], self.weights[layer][name], x, flags)
            b.add(HEAD[1], HEAD[3], HEAD[2], self.logits, self.head_w, self.act_of_layer[-1]["down"], NORM)
            return b
        if flow != "folded":
            raise ValueError(flow)
        if self.res is None:
            rng = np.random.default_rng(777)
            self.res = [GpuBuffer(self.ctx, 4096, np.float32), GpuBuffer(self.ctx, 4096, np.float32)]   # h, h1
            self.gammas = [GpuBuffer.from_host(self.ctx, (np.abs(rng.standard_normal(4096)) + 0.5).astype(np.float32))
                           for _ in range(2)]
        res, gammas = self.res, self.gammas
        for layer in range(self.layers):
            w = self.weights[layer]
            for name in ("q", "k", "v"):
                b.add("q4k", 4096, 4096, act[name], w[name], res[0], NORM, gamma=gammas[0], norm_eps=1e-5)
            b.add("q4k", 4096, 4096, res[1], w["o"], act["q"], 0, residual=res[0])
            for name in ("gate", "up"):
                b.add("q4k", 4096, 11008, act[name], w[name], res[1], NORM, gamma=gammas[1], norm_eps=1e-5)
            b.add("q6k", 11008, 4096, res[0], w["down"], act["gate"], 0, x2=act["up"], residual=res[1])
        b.add(HEAD[1], HEAD[3], HEAD[2], self.logits, self.head_w, res[0], NORM, gamma=gammas[0], norm_eps=1e-5)
        return b
