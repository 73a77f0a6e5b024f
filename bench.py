#!/usr/bin/env python3
"""Benchmark of the k-quant GEMV path on one MI355X.

A step is one 7B-style decode weight pass: 32 layers x {Q,K,V,O: Q4_K 4096x4096; gate, up: Q4_K
11008x4096; down: Q6_K 4096x11008} plus the Q6_K 32000x4096 head - 225 GEMVs over 4.12 GB of
distinct, seeded synthetic weights resident in HBM (far beyond the 256 MB Infinity Cache, so every
pass streams from HBM).  Data flow, per layer: a fresh x_l ~ N(0,1) feeds q, k, v, gate and up; o
consumes the RMS-normalised output of q; down consumes the RMS-normalised output of gate; the head
consumes the RMS-normalised output of the last down.  The list goes to the library in one call, in
layer order (trn_kquant_gemv_batch).  `value` is algorithmic bytes (weights + x + y, each once)
over wall time.  The same 225 GEMVs wired as the strictly serial chain of a decoder (q,k,v <- h;
o <- q; gate,up <- o; down <- gate; h <- down) are timed too and reported in `extra`.

Prints one JSON line.  Extra fields: `roofline` for the dominant kernel (kq_gemv_group: the launches that carry
up to four independent neighbouring entries, 64 per pass, 3.99 of the 4.13 GB), its launches of one pass timed
with HIP events on their stream; `cpu_baseline`: the CPU port
(oracle/cpu_baseline.cpp) on layer 0's seven matrices with all host cores.
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

HBM_PEAK_GBPS = 8000.0
# HBM bytes per kq_gemv_group launch, averaged over the 64 such launches of the full pass: rocprofv3
# FETCH_SIZE and WRITE_SIZE per dispatch, each scaled by what the counter reads for kq_copy_u128 on
# 256 MiB (profiles/kquant_gemv_hbm_traffic_pmc.md).  Counters cannot be read from inside this
# process, so the figure is carried here and re-measured whenever the kernel changes.
GROUP_TRAFFIC_BYTES_PER_LAUNCH = 63_595_450
LAYERS = 32
SB = {"q4k": 144, "q5k": 176, "q6k": 210}
LAYER_MATS = [("q", "q4k", 4096, 4096), ("k", "q4k", 4096, 4096), ("v", "q4k", 4096, 4096), ("o", "q4k", 4096, 4096),
              ("gate", "q4k", 11008, 4096), ("up", "q4k", 11008, 4096), ("down", "q6k", 4096, 11008)]
HEAD = ("head", "q6k", 32000, 4096)


def alg_bytes(fmt, n, k):
    return n * (k // 256) * SB[fmt] + 4 * k + 4 * n


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the single-launch table of configurations 1, 2, 3 and 5")
    ap.add_argument("--no-executors", action="store_true", help="skip the comparison runs of the opt-in one-launch executors")
    ap.add_argument("--layers", type=int, default=LAYERS, help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU; --gpus must be 1 (several GPUs would each take a range of rows of "
              "every matrix and exchange the output vectors)", file=sys.stderr)
        return 2

    import trueno_amd as t
    from oracle import kquant as kq
    from trueno_amd import _ffi

    L = _ffi.lib()
    ctx = t.CudaContext(0)
    stream = t.CudaStream(ctx)
    layers = args.layers

    # ---- seeded synthetic weights, distinct per layer, resident in HBM before timing -------------
    t_gen = time.time()
    weights, xs = [], []
    host_layer0 = {}
    for layer in range(layers):
        mats = {}
        for mi, (name, fmt, n, k) in enumerate(LAYER_MATS):
            host = kq.gen_matrix(fmt, 1234 + 100 * layer + mi, n, k)
            mats[name] = t.GpuBuffer.from_host(ctx, host)
            if layer == 0:
                host_layer0[name] = host
        weights.append(mats)
        xs.append((t.GpuBuffer.from_host(ctx, kq.gen_x(4321 + layer, 4096)),
                   t.GpuBuffer.from_host(ctx, kq.gen_x(8321 + layer, 11008))))
    head_w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(HEAD[1], 999, HEAD[2], HEAD[3]))
    y = {n: t.GpuBuffer(ctx, n, np.float32) for n in (4096, 11008, 32000)}
    ys = {name: t.GpuBuffer(ctx, n, np.float32) for name, _, n, _ in LAYER_MATS}
    print(f"[bench] generated and uploaded {layers} layers in {time.time() - t_gen:.1f} s", file=sys.stderr, flush=True)

    # ---- the pass as one list, in layer order.  Data flow per layer: a fresh x_l ~ N(0,1) feeds q, k, v, gate and
    #      up; o consumes the RMS-normalised output of q; down consumes the RMS-normalised output of gate; the head
    #      consumes the RMS-normalised output of the last down.  The library works out from the pointers which
    #      neighbouring entries are independent of one another.
    NORM = t.GemvBatch.NORM_INPUT
    act = {nm: t.GpuBuffer(ctx, n, np.float32) for nm, n in (("q", 4096), ("k", 4096), ("v", 4096), ("o", 4096),
                                                             ("gate", 11008), ("up", 11008), ("down", 4096))}
    logits = y[32000]
    src_of = {"q": None, "k": None, "v": None, "o": "q", "gate": None, "up": None, "down": "gate"}

    def build_pass(strict):
        """strict: the serial data flow of a decoder (q,k,v <- h; o <- q; gate,up <- o; down <- gate; h <- down)."""
        b = t.GemvBatch()
        nbytes = wbytes = 0
        h = xs[0][0]
        for layer in range(layers):
            for name, fmt, n, k in LAYER_MATS:
                if strict:
                    src = {"q": None, "k": None, "v": None, "o": "q", "gate": "o", "up": "o", "down": "gate"}[name]
                    x, flags = (h if src is None else act[src]), NORM
                else:
                    src = src_of[name]
                    x, flags = (xs[layer][0], 0) if src is None else (act[src], NORM)
                b.add(fmt, k, n, act[name], weights[layer][name], x, flags)
                nbytes += alg_bytes(fmt, n, k)
                wbytes += n * (k // 256) * SB[fmt]
            h = act["down"]
        b.add(HEAD[1], HEAD[3], HEAD[2], logits, head_w, act["down"], NORM)
        nbytes += alg_bytes(HEAD[1], HEAD[2], HEAD[3])
        wbytes += HEAD[2] * (HEAD[3] // 256) * SB[HEAD[1]]
        return b, nbytes, wbytes

    for kv in filter(None, os.environ.get("TRN_BENCH_TUNE", "").split(",")):      # working aid: library tuning keys
        key, val = kv.split("=")
        assert L.trn_set_tuning(key.encode(), int(val)) == 0, kv
    def build_layer_pass():
        """the decoder's serial data flow with the element-wise steps of a layer folded into the entries: q,k,v <-
        rmsnorm(h)*g1; h1 = h + o(q); gate,up <- rmsnorm(h1)*g2; h = h1 + down(silu(gate)*up); head <- rmsnorm(h)*g"""
        b = t.GemvBatch()
        res = [t.GpuBuffer.from_host(ctx, kq.gen_x(777, 4096)), t.GpuBuffer(ctx, 4096, np.float32)]   # h, h1
        gammas = [t.GpuBuffer.from_host(ctx, np.abs(kq.gen_x(780 + i, 4096)) + np.float32(0.5)) for i in range(2)]
        w_of = lambda layer, name: weights[layer][name]
        for layer in range(layers):
            for name in ("q", "k", "v"):
                b.add("q4k", 4096, 4096, act[name], w_of(layer, name), res[0], NORM, gamma=gammas[0], norm_eps=1e-5)
            b.add("q4k", 4096, 4096, res[1], w_of(layer, "o"), act["q"], 0, residual=res[0])
            for name in ("gate", "up"):
                b.add("q4k", 4096, 11008, act[name], w_of(layer, name), res[1], NORM, gamma=gammas[1], norm_eps=1e-5)
            b.add("q6k", 11008, 4096, res[0], w_of(layer, "down"), act["gate"], 0, x2=act["up"], residual=res[1])
        b.add(HEAD[1], HEAD[3], HEAD[2], logits, head_w, res[0], NORM, gamma=gammas[0], norm_eps=1e-5)
        b.keep = (res, gammas)
        return b

    batch, total_bytes, weight_bytes = build_pass(False)
    strict_batch, _, _ = build_pass(True)
    layer_batch = build_layer_pass()

    def ev():
        e = C.c_void_p()
        assert L.trn_event_create(C.byref(e)) == 0
        return e

    # one plain copy of known size (256 MiB read + 256 MiB written): the yardstick that profiler byte
    # counters of the same run are scaled by
    cal_src = t.GpuBuffer(ctx, 64 << 20, np.float32)
    cal_dst = t.GpuBuffer(ctx, 64 << 20, np.float32)
    assert L.trn_copy_u128(stream.raw(), cal_dst.as_ptr(), cal_src.as_ptr(), 256 << 20) == 0
    stream.synchronize()
    cal_src.free()
    cal_dst.free()

    def elapsed_ms(a, b):
        ms = C.c_float()
        assert L.trn_event_elapsed_ms(C.byref(ms), a, b) == 0
        return float(ms.value)

    def run_passes(steps, warmup, batch=batch):
        for _ in range(warmup):
            batch.launch(stream)
        stream.synchronize()
        e0, e1 = ev(), ev()
        t0 = time.perf_counter()
        L.trn_event_record(e0, stream.raw())
        for _ in range(steps):
            batch.launch(stream)
        L.trn_event_record(e1, stream.raw())
        stream.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        return wall / steps, elapsed_ms(e0, e1) / steps

    # ---- timed region: W warm-up passes, then exactly K passes (one cooperative launch per pass) ----
    ms_per_step, gpu_ms_per_step = run_passes(args.steps, args.warmup)
    value = total_bytes / (ms_per_step * 1e-3) / 1e9
    assert np.all(np.isfinite(logits.copy_to_host())), "the pass produced non-finite logits"

    # ---- dominant kernel: kq_gemv_group.  The library puts entries that are independent of one another (and of what
    #      they would overtake) into one launch of this kernel; trn_kquant_gemv_plan says which entry of the pass goes
    #      into which launch.  The launches of the pass that hold two or more entries (all of it but a few single
    #      GEMVs, which take the single-GEMV kernels) are issued here one list each, in pass order, back to back on
    #      the stream, bracketed by HIP events on that stream.
    launch_of = batch.plan()
    members = {}
    for i, l in enumerate(launch_of):
        members.setdefault(l, []).append(i)
    entry_bytes = [alg_bytes(fmt, n, k) for _ in range(layers) for _, fmt, n, k in LAYER_MATS] + [alg_bytes(HEAD[1], HEAD[2], HEAD[3])]
    entry_names = [name for _ in range(layers) for name, _, _, _ in LAYER_MATS] + ["head"]
    kinds = {}
    for l in sorted(members):
        sig = "[" + ",".join(entry_names[i] for i in members[l]) + "]"
        kinds[sig] = kinds.get(sig, 0) + 1
    print("[bench] launches of the pass: " + ", ".join(f"{c} x {sig}" for sig, c in kinds.items()), file=sys.stderr, flush=True)
    groups = []
    grp_bytes = 0
    for l in sorted(members):
        if len(members[l]) >= 2:
            g = batch.subset(members[l])
            assert len(set(g.plan())) == 1, "a launch of the pass, issued alone, must again be one launch"
            groups.append(g)
            grp_bytes += sum(entry_bytes[i] for i in members[l])
    n_grp = len(groups)
    e0, e1 = ev(), ev()
    grp_ms = []
    for _ in range(5):
        for g in groups:
            g.launch(stream)
        stream.synchronize()
        L.trn_event_record(e0, stream.raw())
        for g in groups:
            g.launch(stream)
        L.trn_event_record(e1, stream.raw())
        stream.synchronize()
        grp_ms.append(elapsed_ms(e0, e1) / n_grp)
    grp_ms = sorted(grp_ms)[len(grp_ms) // 2]
    grp_bytes_per_launch = grp_bytes / n_grp
    achieved = grp_bytes_per_launch / (grp_ms * 1e-3) / 1e9

    # ---- the same GEMVs wired as the strictly serial chain of a decoder ------------------------------------
    strict_ms, _ = run_passes(max(3, args.steps // 2), 2, strict_batch)
    layer_ms, _ = run_passes(max(3, args.steps // 2), 2, layer_batch)

    # ---- the same list through the one-launch executors (opt-in), for comparison ------------------------
    other_modes = {}
    for mode, label in (() if args.no_executors else ((1, "resident_phases"),)):
        L.trn_set_tuning(b"batch_mode", mode)
        ms, _ = run_passes(max(3, args.steps // 2), 1)
        other_modes[label] = round(ms * 1e3, 1)
    L.trn_set_tuning(b"batch_mode", 0)

    # ---- per-shape single-launch table (cold: rotates through the layers' copies) -----------------------
    shapes = {}
    for name, fmt, n, k in LAYER_MATS[3:] + [HEAD]:
        b = t.GemvBatch()
        reps = layers if name != "head" else 8
        for r in range(reps):
            wbuf = head_w if name == "head" else weights[r % layers][name]
            b.add(fmt, k, n, y[n], wbuf, xs[r % layers][1 if k == 11008 else 0])
        b.launch(stream)
        stream.synchronize()
        L.trn_event_record(e0, stream.raw())
        b.launch(stream)
        L.trn_event_record(e1, stream.raw())
        stream.synchronize()
        us = elapsed_ms(e0, e1) * 1e3 / reps
        key = f"{fmt}_{n}x{k}" + ("_hot" if name == "head" else "")
        shapes[key] = {"us": round(us, 2), "gbps": round(alg_bytes(fmt, n, k) / us / 1e3, 1),
                       "frac_of_peak": round(alg_bytes(fmt, n, k) / us / 1e3 / HBM_PEAK_GBPS, 4)}

    # ---- the other benchmark configurations, one launch each, cold (16 distinct device copies in rotation) --------
    configs = {}
    if not args.no_configs:
        def timed(launch, reps):
            for r in range(reps):
                launch(r)
            stream.synchronize()
            L.trn_event_record(e0, stream.raw())
            for r in range(reps):
                launch(r)
            L.trn_event_record(e1, stream.raw())
            stream.synchronize()
            return elapsed_ms(e0, e1) * 1e3 / reps

        copies = 16
        for label, fmt, n, k in (("1_q4k_gemv", "q4k", 4096, 4096), ("2_q6k_gemv", "q6k", 4096, 4096),
                                 ("2_q6k_gemv", "q6k", 32000, 4096), ("3_q5k_gemv", "q5k", 11008, 4096),
                                 ("3_q5k_gemv", "q5k", 4096, 11008)):
            host = kq.gen_matrix(fmt, 1234, n, k)
            bufs = [t.GpuBuffer.from_host(ctx, host) for _ in range(copies)]
            xb = xs[0][1 if k == 11008 else 0]
            fn = getattr(L, f"trn_{fmt}_gemv")
            us = timed(lambda r: fn(stream.raw(), y[n].as_ptr(), bufs[r % copies].as_ptr(), xb.as_ptr(), k, n), 2 * copies)
            # the same launch on one copy over and over: the weights come from the 256 MB last-level cache, not from HBM
            hot = timed(lambda r: fn(stream.raw(), y[n].as_ptr(), bufs[0].as_ptr(), xb.as_ptr(), k, n), 2 * copies)
            configs[f"{label}_{n}x{k}"] = {"us": round(us, 2), "gbps": round(alg_bytes(fmt, n, k) / us / 1e3, 1),
                                            "frac_of_peak": round(alg_bytes(fmt, n, k) / us / 1e3 / HBM_PEAK_GBPS, 4),
                                            "us_cache_hot": round(hot, 2)}
            for b in bufs:
                b.free()
        for n, k in ((14336, 4096), (4096, 14336)):
            host = kq.gen_matrix("q4k", 1238, n, k)
            bufs = [t.GpuBuffer.from_host(ctx, host) for _ in range(copies)]
            for m in (1, 4, 16, 64):
                a = t.GpuBuffer.from_host(ctx, kq.gen_x(4321, m, k).reshape(-1))
                c = t.GpuBuffer(ctx, m * n, np.float32)
                us = timed(lambda r: L.trn_q4k_gemm(stream.raw(), a.as_ptr(), bufs[r % copies].as_ptr(), c.as_ptr(), m, n, k),
                           2 * copies)
                nbytes = n * (k // 256) * 144 + 4 * m * k + 4 * m * n
                configs[f"5_q4k_gemm_{n}x{k}_m{m}"] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                                                       "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4),
                                                       "tflops": round(2.0 * m * n * k / us / 1e6, 1)}
                a.free()
                c.free()
            for b in bufs:
                b.free()

        # the GEMM entry points outside BASELINE's configurations: Q5_K / Q6_K (VALU engine per row of A) and the
        # legacy 18-byte format of q4k_gemm_fused, 4096 x 4096, cold
        n = k = 4096
        for fmt in ("q5k", "q6k"):
            host = kq.gen_matrix(fmt, 1239, n, k)
            bufs = [t.GpuBuffer.from_host(ctx, host) for _ in range(copies)]
            fn = getattr(L, f"trn_{fmt}_gemm")
            for m in (4, 16):
                a = t.GpuBuffer.from_host(ctx, kq.gen_x(4321, m, k).reshape(-1))
                c = t.GpuBuffer(ctx, m * n, np.float32)
                us = timed(lambda r: fn(stream.raw(), a.as_ptr(), bufs[r % copies].as_ptr(), c.as_ptr(), m, n, k), 2 * copies)
                nbytes = alg_bytes(fmt, n, k) + 4 * (m - 1) * (k + n)
                configs[f"x_{fmt}_gemm_{n}x{k}_m{m}"] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                                                         "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
                a.free()
                c.free()
            for b in bufs:
                b.free()
        host = kq.gen_q4k_simplified(np.random.default_rng(1240), n * (k // 32))
        bufs = [t.GpuBuffer.from_host(ctx, host) for _ in range(copies)]
        for m in (1, 4):
            a = t.GpuBuffer.from_host(ctx, kq.gen_x(4321, m, k).reshape(-1))
            c = t.GpuBuffer(ctx, m * n, np.float32)
            us = timed(lambda r: L.trn_q4k_gemm_fused(stream.raw(), a.as_ptr(), bufs[r % copies].as_ptr(), c.as_ptr(), m, n, k), 2 * copies)
            nbytes = n * (k // 32) * 18 + 4 * m * (k + n)
            configs[f"x_q4k_gemm_fused_{n}x{k}_m{m}"] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                                                        "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            a.free()
            c.free()
        for b in bufs:
            b.free()

    # ---- the element-wise steps between the GEMVs of a layer, one launch each (latency-bound: a few KB) ----------
    glue_us = {}
    if not args.no_configs:
        hid, ffn = 4096, 11008
        g_a, g_b, g_o, g_g = (t.GpuBuffer.from_host(ctx, kq.gen_x(9000 + i, ffn)) for i in range(4))
        for label, fn in (("residual_add_4096", lambda: L.trn_residual_add(stream.raw(), g_a.as_ptr(), g_b.as_ptr(), g_o.as_ptr(), hid)),
                          ("rmsnorm_4096", lambda: L.trn_rmsnorm(stream.raw(), g_a.as_ptr(), g_o.as_ptr(), g_g.as_ptr(), hid, C.c_float(1e-5))),
                          ("fused_residual_rmsnorm_4096", lambda: L.trn_fused_residual_rmsnorm(
                              stream.raw(), g_a.as_ptr(), g_b.as_ptr(), g_o.as_ptr(), g_g.as_ptr(), hid, C.c_float(1e-5))),
                          ("fused_swiglu_11008", lambda: L.trn_fused_swiglu(stream.raw(), g_a.as_ptr(), g_b.as_ptr(), g_o.as_ptr(), ffn))):
            for _ in range(8):
                fn()
            stream.synchronize()
            L.trn_event_record(e0, stream.raw())
            for _ in range(64):
                fn()
            L.trn_event_record(e1, stream.raw())
            stream.synchronize()
            glue_us[label] = round(elapsed_ms(e0, e1) * 1e3 / 64, 2)

    # ---- the f32 GEMV of gemv.rs (A is K x N row-major), one launch, cold --------------------------------------
    f32_gemv = {}
    if not args.no_configs:
        rng = np.random.default_rng(55)
        for k, n, copies in ((4096, 4096, 8), (4096, 11008, 4)):
            host = rng.standard_normal(k * n, dtype=np.float32)
            bufs = [t.GpuBuffer.from_host(ctx, host) for _ in range(copies)]
            xb, yb = xs[0][0], y[n if n in y else 11008]
            def launch(r):
                return L.trn_gemv_f32(stream.raw(), yb.as_ptr(), bufs[r % copies].as_ptr(), xb.as_ptr(), k, n)
            for r in range(copies):
                launch(r)
            stream.synchronize()
            L.trn_event_record(e0, stream.raw())
            for r in range(2 * copies):
                launch(r)
            L.trn_event_record(e1, stream.raw())
            stream.synchronize()
            us = elapsed_ms(e0, e1) * 1e3 / (2 * copies)
            nbytes = 4 * k * n + 4 * k + 4 * n
            f32_gemv[f"k{k}_n{n}"] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                                      "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            for b in bufs:
                b.free()

    # ---- single-query attention over a KV cache of 7B shape (32 heads x 128), one launch, cold ------------------
    attention = {}
    if not args.no_configs:
        rng = np.random.default_rng(66)
        heads, dim = 32, 128
        for seq in (512, 2048, 8192):
            copies = 6
            kvs = [(t.GpuBuffer.from_host(ctx, rng.standard_normal(heads * seq * dim, dtype=np.float32)),
                    t.GpuBuffer.from_host(ctx, rng.standard_normal(heads * seq * dim, dtype=np.float32))) for _ in range(copies)]
            qb, ob = xs[0][0], y[4096]
            def launch(r):
                return L.trn_incremental_attention(stream.raw(), qb.as_ptr(), kvs[r % copies][0].as_ptr(), kvs[r % copies][1].as_ptr(),
                                                   ob.as_ptr(), seq, dim, heads, heads, seq, C.c_float(dim ** -0.5))
            for r in range(copies):
                assert launch(r) == 0
            stream.synchronize()
            L.trn_event_record(e0, stream.raw())
            for r in range(2 * copies):
                launch(r)
            L.trn_event_record(e1, stream.raw())
            stream.synchronize()
            us = elapsed_ms(e0, e1) * 1e3 / (2 * copies)
            nbytes = 8 * heads * seq * dim + 8 * heads * dim
            attention[f"seq{seq}"] = {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1),
                                      "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}
            for a, b in kvs:
                a.free()
                b.free()

    # ---- a whole decode step: the serial layer chain with folded glue AND attention over a KV cache of 2048 -------
    decode_step = None
    if not args.no_configs:
        heads, dim, seq = 32, 128, 2048
        rng = np.random.default_rng(77)
        kv_host = rng.standard_normal(heads * seq * dim, dtype=np.float32)
        caches = [(t.GpuBuffer.from_host(ctx, kv_host), t.GpuBuffer.from_host(ctx, kv_host)) for _ in range(layers)]
        h0, h1 = t.GpuBuffer.from_host(ctx, kq.gen_x(778, 4096)), t.GpuBuffer(ctx, 4096, np.float32)
        gam = t.GpuBuffer.from_host(ctx, np.abs(kq.gen_x(779, 4096)) + np.float32(0.5))
        attn_out = t.GpuBuffer(ctx, 4096, np.float32)
        pre, post = [], []
        for layer in range(layers):
            a, b = t.GemvBatch(), t.GemvBatch()
            for name in ("q", "k", "v"):
                a.add("q4k", 4096, 4096, act[name], weights[layer][name], h0, NORM, gamma=gam, norm_eps=1e-5)
            b.add("q4k", 4096, 4096, h1, weights[layer]["o"], attn_out, 0, residual=h0)
            for name in ("gate", "up"):
                b.add("q4k", 4096, 11008, act[name], weights[layer][name], h1, NORM, gamma=gam, norm_eps=1e-5)
            b.add("q6k", 11008, 4096, h0, weights[layer]["down"], act["gate"], 0, x2=act["up"], residual=h1)
            pre.append(a)
            post.append(b)
        head_b = t.GemvBatch().add(HEAD[1], HEAD[3], HEAD[2], logits, head_w, h0, NORM, gamma=gam, norm_eps=1e-5)

        def step():
            for layer in range(layers):
                pre[layer].launch(stream)
                L.trn_incremental_attention(stream.raw(), act["q"].as_ptr(), caches[layer][0].as_ptr(), caches[layer][1].as_ptr(),
                                            attn_out.as_ptr(), seq, dim, heads, heads, seq, C.c_float(dim ** -0.5))
                post[layer].launch(stream)
            head_b.launch(stream)
        step()
        stream.synchronize()
        L.trn_event_record(e0, stream.raw())
        for _ in range(3):
            step()
        L.trn_event_record(e1, stream.raw())
        stream.synchronize()
        us = elapsed_ms(e0, e1) * 1e3 / 3
        kv_bytes = layers * (8 * heads * seq * dim)
        decode_step = {"us": round(us, 1), "kv_positions": seq, "weight_bytes": weight_bytes, "kv_cache_bytes": kv_bytes,
                       "gbps": round((total_bytes + kv_bytes) / us / 1e3, 1)}
        for a, b in caches:
            a.free()
            b.free()

    # ---- CPU baseline: the port, layer 0's seven matrices, all host cores --------------------------
    cpu = None
    cpu_config1 = None
    if not args.no_cpu_baseline:
        from oracle.cref import CpuBaseline
        cb = CpuBaseline()
        # the GPU box gives this job a share of the host's cores; do not oversubscribe it
        cores = max(1, min(cb.threads(), int(os.environ.get("OMP_NUM_THREADS", cb.threads()))))
        hx = {4096: kq.gen_x(4321, 4096), 11008: kq.gen_x(8321, 11008)}
        layer_bytes = sum(alg_bytes(fmt, n, k) for _, fmt, n, k in LAYER_MATS)
        reps, spent = 0, 0.0
        t_start = time.time()
        while (spent < 10.0 and reps < 4000) or reps < 2:      # about 10 s of wall time on all the job's cores
            for name, fmt, n, k in LAYER_MATS:
                _, sec = cb.dequant_matvec(fmt, host_layer0[name], hx[k], k, n, cores, 1)
                spent += sec
            reps += 1
            if time.time() - t_start > 40:
                break
        # configuration 1 on the CPU path: dequantise + matvec per call, and matvec on weights dequantised beforehand
        n1 = k1 = 4096
        _, sec_dq = cb.dequant_matvec("q4k", host_layer0["q"], hx[k1], k1, n1, cores, 5)
        w_f32 = kq.dequant_matrix("q4k", host_layer0["q"], n1, k1)
        _, sec_mv = cb.matvec_f32(w_f32, hx[k1], cores, 5)
        cpu_config1 = {"shape": "Q4_K 4096x4096", "cores": cores,
                       "dequant_matvec_us": round(sec_dq / 5 * 1e6, 1),
                       "dequant_matvec_gbps_quantized": round(alg_bytes("q4k", n1, k1) / (sec_dq / 5) / 1e9, 2),
                       "matvec_predequantised_f32_us": round(sec_mv / 5 * 1e6, 1),
                       "matvec_predequantised_gbps_quantized": round(alg_bytes("q4k", n1, k1) / (sec_mv / 5) / 1e9, 2)}
        # configurations 2 and 3 on the CPU path (dequantise + matvec per call)
        for label, fmt, n, k in (("2_q6k_4096x4096", "q6k", 4096, 4096), ("2_q6k_32000x4096", "q6k", 32000, 4096),
                                 ("3_q5k_11008x4096", "q5k", 11008, 4096), ("3_q5k_4096x11008", "q5k", 4096, 11008)):
            wm = kq.gen_matrix(fmt, 1234 + n + k, n, k)
            _, sec = cb.dequant_matvec(fmt, wm, hx[k], k, n, cores, 3)
            cpu_config1[label] = {"dequant_matvec_us": round(sec / 3 * 1e6, 1),
                                  "dequant_matvec_gbps_quantized": round(alg_bytes(fmt, n, k) / (sec / 3) / 1e9, 2)}
        cpu = {"value": round(layer_bytes * reps / spent / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"layer 0 of the pass (7 GEMVs, {layer_bytes / 1e6:.1f} MB quantized) x {reps} repetitions, "
                         f"dequantise-row + AVX2 dot, {'AVX2+FMA' if cb.has_avx2() else 'scalar'}"}

    out = {
        "metric": "k-quant GEMV achieved HBM GB/s (% of peak) + \u00b5s per 7B decode weight pass",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"7B-style decode weight pass: {layers} layers x (4x Q4_K 4096x4096 + 2x Q4_K 11008x4096 + "
                               f"1x Q6_K 4096x11008) + Q6_K 32000x4096 head; {len(batch)} GEMVs in layer order "
                               f"(per layer x_l~N(0,1) -> q,k,v,gate,up; o<-norm(q); down<-norm(gate); head<-norm(down)), "
                               f"{total_bytes / 1e9:.3f} GB, batch 1, f32 x and y", "gemvs": len(batch),
                               "bytes_per_step": total_bytes},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": GROUP_TRAFFIC_BYTES_PER_LAUNCH if layers == LAYERS else None,
                     "kernel": "kq_gemv_group", "launches_per_pass": n_grp,
                     "bytes_per_launch": round(grp_bytes_per_launch), "us_per_launch": round(grp_ms * 1e3, 3)},
        "cpu_baseline": cpu,
        "extra": {"us_per_pass": round(ms_per_step * 1e3, 1), "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
                  "gpu_event_us_per_pass": round(gpu_ms_per_step * 1e3, 1),
                  "us_per_pass_strict_decoder_chain": round(strict_ms * 1e3, 1),
                  "us_per_pass_one_launch_executors": other_modes,
                  "weight_bytes": weight_bytes, "us_per_pass_decoder_chain_with_folded_layer_glue": round(layer_ms * 1e3, 1),
                  "per_shape_single_launch_cold": shapes, "layer_glue_us_per_launch_back_to_back": glue_us, "decode_step_7b_folded_glue_and_attention": decode_step, "f32_gemv_single_launch_cold": f32_gemv, "incremental_attention_32x128_single_launch_cold": attention,
                  "other_configs_single_launch_cold": configs, "cpu_config1": cpu_config1,
                  "device": ctx.device_name(), "cus": ctx.cu_count()},
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
