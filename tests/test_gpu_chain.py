"""GPU parity, the list executor (trn_kquant_gemv_batch): dependent chains of GEMVs with the optional
input normalisation, checked entry by entry against fp64 on each entry's ACTUAL input, against the
one-launch-per-entry path (bit for bit), across repeated launches, and through its bounded-wait
abort path."""
import ctypes as C

import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import _ffi

pytestmark = pytest.mark.gpu
TOL = 1e-5
EPS = 1e-6


@pytest.fixture(autouse=True)
def resident_mode():
    """these tests exercise the resident-workgroup form of the executor unless they say otherwise"""
    _ffi.lib().trn_set_tuning(b"batch_mode", 1)
    yield
    _ffi.lib().trn_set_tuning(b"batch_mode", 0)


def _tune(key, value):
    assert _ffi.lib().trn_set_tuning(key.encode(), int(value)) == 0


class Chain:
    """host model of a list: buffers by name, entries (fmt, n, k, w_host, x_name, y_name, flags)"""

    def __init__(self, gpu):
        self.ctx, self.stream = gpu
        self.bufs, self.entries, self.batch = {}, [], t.GemvBatch()

    def buffer(self, name, data_or_len):
        if isinstance(data_or_len, int):
            self.bufs[name] = t.GpuBuffer.from_host(self.ctx, np.full(data_or_len, np.nan, np.float32))
        else:
            self.bufs[name] = t.GpuBuffer.from_host(self.ctx, np.ascontiguousarray(data_or_len, np.float32))
        return self.bufs[name]

    def add(self, fmt, n, k, seed, x_name, y_name, flags=0):
        host = kq.gen_matrix(fmt, seed, n, k)
        dw = t.GpuBuffer.from_host(self.ctx, host)
        self.entries.append((fmt, n, k, host, dw, x_name, y_name, flags))
        self.batch.add(fmt, k, n, self.bufs[y_name], dw, self.bufs[x_name], flags)

    def run(self):
        self.batch.launch(self.stream)
        self.stream.synchronize()
        return {k: v.copy_to_host() for k, v in self.bufs.items()}

    def check(self, out, initial):
        """replay in order on the host: each entry's fp64 result from the GPU's own input values"""
        state = {k: v.copy() for k, v in initial.items()}
        worst = 0.0
        for fmt, n, k, host, _, xn, yn, flags in self.entries:
            x = state[xn][:k].astype(np.float64)
            if flags & 1:
                x = x / np.sqrt(np.mean(x * x) + EPS)
            y64 = kq.dequant_matrix(fmt, host, n, k).astype(np.float64) @ x
            state[yn] = state[yn].copy()
            # what the GPU produced for this entry is what later entries consumed
            got = self.final_or_intermediate(out, yn)
            if got is not None:
                err = kq.rel_l2(got[:n], y64)
                worst = max(worst, err)
                assert err <= TOL, (fmt, n, k, err)
                state[yn][:n] = got[:n]
            else:
                state[yn][:n] = y64.astype(np.float32)
        return worst

    def final_or_intermediate(self, out, name):
        return out.get(name)


def test_chain_dependent_layers_match_fp64_and_per_launch_path(gpu):
    """two 'layers' in the shape of a decoder block (small sizes): QKV <- h, O <- q, gate/up <- o, down <- gate;
    every output buffer is written once, so every intermediate can be checked on its actual input"""
    h0 = kq.gen_x(1, 1024)

    def build():
        c = Chain(gpu)
        c.buffer("h0", h0)
        prev = "h0"
        for layer in range(2):
            for nm, n in (("q", 1024), ("k", 1024), ("v", 1024), ("o", 1024), ("g", 2816), ("u", 2816), ("d", 1024)):
                c.buffer(f"{nm}{layer}", n)
            s = 100 * layer
            c.add("q4k", 1024, 1024, s + 1, prev, f"q{layer}", 1)
            c.add("q4k", 1024, 1024, s + 2, prev, f"k{layer}", 1)
            c.add("q5k", 1024, 1024, s + 3, prev, f"v{layer}", 1)
            c.add("q4k", 1024, 1024, s + 4, f"q{layer}", f"o{layer}", 1)
            c.add("q4k", 2816, 1024, s + 5, f"o{layer}", f"g{layer}", 1)
            c.add("q5k", 2816, 1024, s + 6, f"o{layer}", f"u{layer}", 1)
            c.add("q6k", 1024, 2816, s + 7, f"g{layer}", f"d{layer}", 1)
            prev = f"d{layer}"
        return c

    _tune("batch_mode", 1)
    c = build()
    out = c.run()
    init = {k: np.full(v.size, np.nan, np.float32) for k, v in out.items()}
    init["h0"] = h0
    worst = c.check(out, init)
    assert all(np.all(np.isfinite(v)) for v in out.values())
    # second and third launch of the same list (counters are reset per launch; the list is not re-uploaded)
    for _ in range(2):
        again = c.run()
        for k in out:
            assert np.array_equal(out[k].view(np.uint32), again[k].view(np.uint32)), k
    # one launch per entry gives the same bits
    _tune("batch_mode", 0)
    ref = build().run()
    for k in out:
        assert np.array_equal(out[k].view(np.uint32), ref[k].view(np.uint32)), k
    print(f"chain worst rel-L2 vs fp64 on actual inputs: {worst:.3e}")


def test_chain_real_shapes_one_layer(gpu):
    """one layer at the 7B shapes plus the head, dependent, normalised"""
    c = Chain(gpu)
    h = kq.gen_x(5, 4096)
    c.buffer("h", h)
    for nm, n in (("q", 4096), ("k", 4096), ("v", 4096), ("o", 4096), ("g", 11008), ("u", 11008), ("d", 4096), ("logits", 32000)):
        c.buffer(nm, n)
    c.add("q4k", 4096, 4096, 11, "h", "q", 1)
    c.add("q4k", 4096, 4096, 12, "h", "k", 1)
    c.add("q4k", 4096, 4096, 13, "h", "v", 1)
    c.add("q4k", 4096, 4096, 14, "q", "o", 1)
    c.add("q4k", 11008, 4096, 15, "o", "g", 1)
    c.add("q4k", 11008, 4096, 16, "o", "u", 1)
    c.add("q6k", 4096, 11008, 17, "g", "d", 1)
    c.add("q6k", 32000, 4096, 18, "d", "logits", 1)
    out = c.run()
    init = {k: np.full(v.size, np.nan, np.float32) for k, v in out.items()}
    init["h"] = h
    c.check(out, init)


def test_chain_hazards_and_in_place_reuse(gpu):
    """buffers reused along the list: read-after-write, write-after-read and write-after-write all order correctly"""
    ctx, stream = gpu
    k = n = 512
    x0 = kq.gen_x(9, k)
    a, b = t.GpuBuffer.from_host(ctx, x0), t.GpuBuffer.from_host(ctx, np.zeros(n, np.float32))
    mats = [kq.gen_matrix("q4k", 60 + i, n, k) for i in range(6)]
    dws = [t.GpuBuffer.from_host(ctx, m) for m in mats]
    batch = t.GemvBatch()
    ping, pong = a, b
    for i in range(6):                      # a -> b -> a -> b ... each step reads what the previous one wrote
        batch.add("q4k", k, n, pong, dws[i], ping, 1)
        ping, pong = pong, ping
    batch.launch(stream)
    stream.synchronize()
    x = x0.astype(np.float64)
    for i in range(6):
        xn = x / np.sqrt(np.mean(x * x) + EPS)
        x = kq.dequant_matrix("q4k", mats[i], n, k).astype(np.float64) @ xn
    got = ping.copy_to_host()
    assert kq.rel_l2(got, x) <= 5e-5      # six roundings deep; each step is checked on actual inputs elsewhere


def test_chain_without_norm_equals_typed_launchers(gpu):
    ctx, stream = gpu
    n, k = 700, 2048
    x = t.GpuBuffer.from_host(ctx, kq.gen_x(3, k))
    batch, refs = t.GemvBatch(), []
    for fmt, kern, seed in (("q4k", t.Q4KGemvKernel, 1), ("q5k", t.Q5KGemvKernel, 2), ("q6k", t.Q6KGemvKernel, 3)):
        w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(fmt, seed, n, k))
        y1, y2 = t.GpuBuffer(ctx, n, np.float32), t.GpuBuffer(ctx, n, np.float32)
        batch.add(fmt, k, n, y1, w, x)
        kern(k, n).launch(stream, y2, w, x)
        refs.append((y1, y2, w))
    batch.launch(stream)
    stream.synchronize()
    for y1, y2, _ in refs:
        assert np.array_equal(y1.copy_to_host().view(np.uint32), y2.copy_to_host().view(np.uint32))


def test_chain_misaligned_entry_falls_back_to_per_entry_launches(gpu):
    ctx, stream = gpu
    n, k = 300, 1024
    buf, xh = kq.gen_matrix("q4k", 5, n, k), kq.gen_x(6, k)
    w = t.GpuBuffer(ctx, buf.size + 1, np.uint8)
    w.copy_from_host_at(buf, 1)
    x = t.GpuBuffer.from_host(ctx, xh)
    y1, y2 = t.GpuBuffer(ctx, n, np.float32), t.GpuBuffer(ctx, n, np.float32)
    t.GemvBatch().add("q4k", k, n, y1, w.as_ptr() + 1, x, 1).add("q4k", k, n, y2, w.as_ptr() + 1, y1.as_ptr() if False else x, 0).launch(stream)
    stream.synchronize()
    wd = kq.dequant_matrix("q4k", buf, n, k).astype(np.float64)
    x64 = xh.astype(np.float64)
    assert kq.rel_l2(y2.copy_to_host(), wd @ x64) <= TOL
    assert kq.rel_l2(y1.copy_to_host(), wd @ (x64 / np.sqrt(np.mean(x64 * x64) + EPS))) <= TOL


def test_chain_rejects_bad_entries(gpu):
    L = _ffi.lib()
    ctx, stream = gpu
    d = (_ffi.GemvDesc * 2)(_ffi.GemvDesc(4, 256, 4, 0, 16, 16, 16), _ffi.GemvDesc(7, 256, 4, 0, 16, 16, 16))
    assert L.trn_kquant_gemv_batch(stream.raw(), d, 2) == 1
    d[1] = _ffi.GemvDesc(4, 100, 4, 0, 16, 16, 16)
    assert L.trn_kquant_gemv_batch(stream.raw(), d, 2) == 1
    d[1] = _ffi.GemvDesc(4, 256, 4, 16, 16, 16, 16)
    assert L.trn_kquant_gemv_batch(stream.raw(), d, 2) == 1
    assert L.trn_kquant_gemv_batch(stream.raw(), None, 0) == 0


def test_chain_barrier_wait_is_bounded(gpu):
    """a spin budget of one poll makes the device-side waits give up: the kernel exits (no hang), the
    synchronisation that follows reports it once (unless every wait happened to be satisfied at its first poll), and
    normal operation resumes"""
    ctx, stream = gpu
    L = _ffi.lib()
    n = k = 4096
    x = t.GpuBuffer.from_host(ctx, kq.gen_x(1, k))
    ws = [t.GpuBuffer.from_host(ctx, kq.gen_matrix("q4k", 70 + i, n, k)) for i in range(4)]
    ys = [t.GpuBuffer(ctx, n, np.float32) for _ in range(4)]
    batch = t.GemvBatch()
    src = x
    for i in range(4):
        batch.add("q4k", k, n, ys[i], ws[i], src, 1)
        src = ys[i]
    batch.launch(stream)
    stream.synchronize()
    good = ys[3].copy_to_host()
    _tune("chain_spin_limit", 1)
    reported = False
    try:
        batch.launch(stream)
        stream.synchronize()         # the call that says "done" reports the abandoned wait, once
    except t.GpuError as e:
        reported = True
        assert e.code == 9001 and "WAIT_ABANDONED" in str(e)
    finally:
        _tune("chain_spin_limit", 0)
    stream.synchronize()             # reported once: the stream is usable and clean again
    batch.launch(stream)
    stream.synchronize()
    assert np.array_equal(ys[3].copy_to_host().view(np.uint32), good.view(np.uint32))
    print("barrier abort reported:", reported)
