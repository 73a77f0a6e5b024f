"""GPU parity: GEMV list entries with the element-wise steps of a decoder layer folded in (rmsnorm with gamma in front of
a projection, swiglu in front of the down projection, the residual add behind o and down), through the C ABI.

Every entry is checked in fp64 on the values the GPU actually fed it, to the GEMV tolerance (1e-5 relative L2); the
folded list is also checked against the same layer done with the stand-alone element-wise kernels, and the three ways of
issuing a list must agree bit for bit."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import glue
from oracle import kquant as kq
from trueno_amd import _ffi

pytestmark = pytest.mark.gpu
TOL = 1e-5
HID, FFN, EPS = 512, 1024, 1e-5


def _tune(key, value):
    assert _ffi.lib().trn_set_tuning(key.encode(), int(value)) == 0


class Layer:
    """one decoder layer without attention: q,k,v <- rmsnorm(h)*g1; h1 = h + o(q); gate,up <- rmsnorm(h1)*g2;
    h2 = h1 + down(silu(gate)*up)"""

    SHAPES = (("q", "q4k", HID, HID), ("k", "q4k", HID, HID), ("v", "q6k", HID, HID), ("o", "q4k", HID, HID),
              ("gate", "q4k", FFN, HID), ("up", "q5k", FFN, HID), ("down", "q6k", HID, FFN))

    def __init__(self, gpu, seed=0):
        self.ctx, self.stream = gpu
        rng = np.random.default_rng(seed)
        self.host = {"h": kq.gen_x(seed + 1, HID), "g1": rng.uniform(0.5, 1.5, HID).astype(np.float32),
                     "g2": rng.uniform(0.5, 1.5, HID).astype(np.float32)}
        self.w_host = {nm: kq.gen_matrix(fmt, seed + 10 + i, n, k) for i, (nm, fmt, n, k) in enumerate(self.SHAPES)}
        self.w = {nm: t.GpuBuffer.from_host(self.ctx, self.w_host[nm]) for nm in self.w_host}
        self.fmt = {nm: fmt for nm, fmt, _, _ in self.SHAPES}

    def fresh(self):
        b = {nm: t.GpuBuffer.from_host(self.ctx, np.full(n, np.nan, np.float32)) for nm, _, n, _ in self.SHAPES}
        for nm in ("h", "g1", "g2"):
            b[nm] = t.GpuBuffer.from_host(self.ctx, self.host[nm])
        b["h1"] = t.GpuBuffer.from_host(self.ctx, np.full(HID, np.nan, np.float32))
        b["h2"] = t.GpuBuffer.from_host(self.ctx, np.full(HID, np.nan, np.float32))
        return b

    def folded(self, b):
        N = t.GemvBatch.NORM_INPUT
        batch = t.GemvBatch()
        for nm in ("q", "k", "v"):
            batch.add(self.fmt[nm], HID, HID, b[nm], self.w[nm], b["h"], N, gamma=b["g1"], norm_eps=EPS)
        batch.add("q4k", HID, HID, b["h1"], self.w["o"], b["q"], 0, residual=b["h"])
        batch.add("q4k", HID, FFN, b["gate"], self.w["gate"], b["h1"], N, gamma=b["g2"], norm_eps=EPS)
        batch.add("q5k", HID, FFN, b["up"], self.w["up"], b["h1"], N, gamma=b["g2"], norm_eps=EPS)
        batch.add("q6k", FFN, HID, b["h2"], self.w["down"], b["gate"], 0, x2=b["up"], residual=b["h1"])
        return batch

    def run_folded(self):
        b = self.fresh()
        batch = self.folded(b)
        batch.launch(self.stream)
        self.stream.synchronize()
        return {k: v.copy_to_host() for k, v in b.items()}

    def run_unfolded(self):
        """the same layer with the stand-alone kernels between plain GEMVs"""
        b, s = self.fresh(), self.stream
        tmp = t.GpuBuffer(self.ctx, max(HID, FFN), np.float32)
        t.RmsNormKernel(HID).with_epsilon(EPS).launch(s, b["h"], tmp, b["g1"])
        for nm, K in (("q", t.Q4KGemvKernel), ("k", t.Q4KGemvKernel), ("v", t.Q6KGemvKernel)):
            K(HID, HID).launch(s, b[nm], self.w[nm], tmp)
        t.Q4KGemvKernel(HID, HID).launch(s, b["o"], self.w["o"], b["q"])
        t.ResidualAddKernel(HID).launch(s, b["h"], b["o"], b["h1"])
        t.RmsNormKernel(HID).with_epsilon(EPS).launch(s, b["h1"], tmp, b["g2"])
        t.Q4KGemvKernel(HID, FFN).launch(s, b["gate"], self.w["gate"], tmp)
        t.Q5KGemvKernel(HID, FFN).launch(s, b["up"], self.w["up"], tmp)
        t.FusedSwigluKernel(FFN).launch(s, b["gate"], b["up"], tmp)
        t.Q6KGemvKernel(FFN, HID).launch(s, b["down"], self.w["down"], tmp)
        t.ResidualAddKernel(HID).launch(s, b["h1"], b["down"], b["h2"])
        s.synchronize()
        return {k: v.copy_to_host() for k, v in b.items()}

    def check_fp64(self, out):
        """each entry in fp64 from the GPU's own inputs"""
        W = {nm: kq.dequant_matrix(fmt, self.w_host[nm], n, k).astype(np.float64) for nm, fmt, n, k in self.SHAPES}
        h = self.host["h"]
        worst = 0.0
        for nm in ("q", "k", "v"):
            worst = max(worst, kq.rel_l2(out[nm], W[nm] @ glue.rmsnorm_fp64(h, self.host["g1"], EPS)))
        worst = max(worst, kq.rel_l2(out["h1"], h.astype(np.float64) + W["o"] @ out["q"].astype(np.float64)))
        x = glue.rmsnorm_fp64(out["h1"], self.host["g2"], EPS)
        worst = max(worst, kq.rel_l2(out["gate"], W["gate"] @ x), kq.rel_l2(out["up"], W["up"] @ x))
        act = glue.fused_swiglu_fp64(out["gate"], out["up"])
        worst = max(worst, kq.rel_l2(out["h2"], out["h1"].astype(np.float64) + W["down"] @ act))
        return worst


def test_folded_layer_matches_fp64_and_the_stand_alone_kernels(gpu):
    layer = Layer(gpu, 5)
    folded = layer.run_folded()
    worst = layer.check_fp64(folded)
    print(f"folded layer: worst relative L2 against fp64 {worst:.3e}")
    assert worst <= TOL
    plain = layer.run_unfolded()
    for nm in ("q", "k", "v", "h1", "gate", "up", "h2"):
        assert kq.rel_l2(folded[nm], plain[nm].astype(np.float64)) <= 2 * TOL, nm


def test_folded_layer_is_the_same_bits_however_the_list_is_issued(gpu):
    layer = Layer(gpu, 6)
    ref = layer.run_folded()
    try:
        _tune("group_off", 1)
        ungrouped = layer.run_folded()
    finally:
        _tune("group_off", 0)
    try:
        _tune("batch_mode", 1)
        phases = layer.run_folded()
    finally:
        _tune("batch_mode", 0)
    for nm in ("q", "k", "v", "h1", "gate", "up", "h2"):
        for other, label in ((ungrouped, "one launch per entry"), (phases, "resident phases")):
            assert np.array_equal(ref[nm].view(np.uint32), other[nm].view(np.uint32)), (nm, label)


def test_residual_in_place_and_bad_folded_entries(gpu):
    ctx, stream = gpu
    n = k = 512
    host = kq.gen_matrix("q4k", 77, n, k)
    w = t.GpuBuffer.from_host(ctx, host)
    x, h = kq.gen_x(78, k), kq.gen_x(79, n)
    dx, dh = t.GpuBuffer.from_host(ctx, x), t.GpuBuffer.from_host(ctx, h)
    t.GemvBatch().add("q4k", k, n, dh, w, dx, residual=dh).launch(stream)          # h += W x
    stream.synchronize()
    want = h.astype(np.float64) + kq.dequant_matrix("q4k", host, n, k).astype(np.float64) @ x.astype(np.float64)
    assert kq.rel_l2(dh.copy_to_host(), want) <= TOL
    L = _ffi.lib()
    bad = _ffi.GemvDesc(4, k, n, 8, dh.as_ptr(), w.as_ptr(), dx.as_ptr(), 0, 0, 0, 0.0, 0)     # swiglu flag without x2
    assert L.trn_kquant_gemv_batch(stream.raw(), (_ffi.GemvDesc * 1)(bad), 1) == 1
    bad = _ffi.GemvDesc(4, k, n, 0, dh.as_ptr(), w.as_ptr(), dx.as_ptr(), dx.as_ptr() + 4, 0, 0, 0.0, 0)   # gamma not 16-byte aligned
    assert L.trn_kquant_gemv_batch(stream.raw(), (_ffi.GemvDesc * 1)(bad), 1) == 1
