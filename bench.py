#!/usr/bin/env python3
"""Benchmark of the k-quant GEMV path on one MI355X.

A step is one 7B-style decode weight pass: 32 layers x {Q,K,V,O: Q4_K 4096x4096; gate, up: Q4_K
11008x4096; down: Q6_K 4096x11008} plus the Q6_K 32000x4096 head - 225 GEMVs over 4.12 GB of
distinct, seeded synthetic weights resident in HBM (far beyond the 256 MB Infinity Cache, so every
pass streams from HBM).  Data flow, per layer: a fresh x_l ~ N(0,1) feeds q, k, v, gate and up; o
consumes the RMS-normalised output of q; down consumes the RMS-normalised output of gate; the head
consumes the RMS-normalised output of the last down.  Every layer writes activation buffers of its own,
so nothing but that data flow orders the entries (with one set of buffers shared by all layers, as a
decoder's are, a layer's q must also wait until the previous layer's o has read it: that pass is timed
too, `same_pass_with_shared_activation_buffers` in `config`).  The list (trueno_amd.decode_pass, the one
the GPU parity test checks) goes to the library in one call, in layer order (trn_kquant_gemv_batch).
`value` is algorithmic bytes (weights + x + y, each once) over wall time.  After the timed region the
last layer's outputs and the logits are checked against fp64 on their actual inputs.  The same 225
GEMVs wired as the strictly serial chain of a decoder (q,k,v <- h; o <- q; gate,up <- o; down <- gate;
h <- down) are timed too: `strict_decoder_chain` in `config`.

Prints one JSON line.  `per_pass_us` (in `extra`): minimum, median and maximum of the K timed passes (and all K in order), from one HIP event
between consecutive passes of the timed region itself.  `roofline`: the dominant kernel, kq_gemv_many (the two launches
of a pass that take their many entries from tables in device memory: the 160 q, k, v, gate, up matrices, then the 64 o and
down matrices; the head alone runs kq_gemv_group).  Its launches are timed with HIP events on their stream in a second
region of the same K passes after the same W warm-up passes, each pass issued as its launches one list each with an event
between them; that region's time per pass is reported beside the headline's.  `bare_read_*`: a launch that only reads as
many bytes (non-temporal 16-byte loads, whole lines once), same protocol.  `cpu_baseline`: the CPU port
(oracle/cpu_baseline.cpp) on layer 0's seven matrices with all host cores.  `extra` holds the other benchmark
configurations, timed as launches back to back over at least 1 GiB of distinct copies (200 launches, median of 5
batches), one copy over and over ("hot": from the last-level cache), and eight independent copies per library call (the
grouped launch in steady state).  A 4 KB read (kq_read_u128 with one workgroup) is launched just outside each of the two
regions: in a kernel trace it marks where they begin and end (rocprof_summary.py timed).
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
TOL = 1e-5                      # relative L2 against fp64, as in the parity tests
GIB = 1 << 30
# HBM bytes per kq_gemv_group launch as the hardware counters saw them: written next to the rocprofv3 summaries by
# the script that makes them (python rocprof_summary.py), with the commit it was measured at.
TRAFFIC_JSON = os.path.join(ROOT, "profiles", "kquant_gemv_many_traffic.json")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=40,
                    help="untimed passes first (a pass is 0.7 ms and the clocks take some 20 ms of load to settle: with 10 warm-up passes the "
                         "first 14 timed ones still fell from 850 to 720 us)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true", help="skip the tables of configurations 1, 2, 3 and 5 and of the path's neighbours")
    ap.add_argument("--executors", action="store_true", help="also time the opt-in one-launch executor (batch_mode 1; slower than launches on every list)")
    ap.add_argument("--pass-only", action="store_true",
                    help="only the timed passes and the launches of the roofline figure (for counter runs: every dispatch of the "
                         "dominant kernel then belongs to the pass)")
    args = ap.parse_args()
    if args.pass_only:
        args.no_cpu_baseline = args.no_configs = True
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU; --gpus must be 1 (several GPUs would each take a range of rows of "
              "every matrix and exchange the output vectors)", file=sys.stderr)
        return 2

    import trueno_amd as t
    from oracle import kquant as kq
    from trueno_amd import _ffi
    from trueno_amd.decode_pass import HEAD, LAYER_MATS, SB, DecodePass, alg_bytes

    L = _ffi.lib()
    ctx = t.CudaContext(0)
    stream = t.CudaStream(ctx)
    layers = 32

    # ---- seeded synthetic weights, distinct per layer, resident in HBM before timing -------------
    t_gen = time.time()
    weights, xs, host_layer0, host_last = [], [], {}, {}
    for layer in range(layers):
        mats = {}
        for mi, (name, fmt, n, k) in enumerate(LAYER_MATS):
            host = kq.gen_matrix(fmt, 1234 + 100 * layer + mi, n, k)
            mats[name] = t.GpuBuffer.from_host(ctx, host)
            if layer == 0:
                host_layer0[name] = host
            if layer == layers - 1:
                host_last[name] = host
        weights.append(mats)
        xs.append(kq.gen_x(4321 + layer, 4096))
    host_head = kq.gen_matrix(HEAD[1], 999, HEAD[2], HEAD[3])
    dp = DecodePass(ctx, weights, t.GpuBuffer.from_host(ctx, host_head), [t.GpuBuffer.from_host(ctx, x) for x in xs])
    x11008 = t.GpuBuffer.from_host(ctx, kq.gen_x(8321, 11008))
    y = {n: t.GpuBuffer(ctx, n, np.float32) for n in (4096, 11008, 14336, 32000)}
    print(f"[bench] generated and uploaded {layers} layers in {time.time() - t_gen:.1f} s", file=sys.stderr, flush=True)

    batch, shared_batch = dp.build("fresh_x_own_buffers"), dp.build("fresh_x")
    strict_batch, layer_batch = dp.build("strict"), dp.build("folded")
    entry_bytes, entry_names = dp.entry_bytes(), dp.entry_names()
    total_bytes, weight_bytes = sum(entry_bytes), dp.weight_bytes()
    act, logits, head_w = dp.act, dp.logits, dp.head_w
    NORM = t.GemvBatch.NORM_INPUT

    def ev():
        e = C.c_void_p()
        assert L.trn_event_create(C.byref(e)) == 0
        return e

    e0, e1 = ev(), ev()

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

    mark = t.GpuBuffer(ctx, 2048, np.float32)

    def region_mark():
        # a 4 KB read: in a kernel trace it separates what follows from what came before
        L.trn_read_u128(stream.raw(), mark.as_ptr(), 4096, mark.as_ptr() + 4096)

    pass_events = [ev() for _ in range(args.steps + 1)]

    def run_passes(steps, warmup, batch=batch, events=None, marks=False):
        """W untimed passes, then exactly K: wall clock per pass between two synchronisations, and the device's own time per
        pass between the events around the K passes.  events: K + 1 events, one recorded between consecutive passes."""
        for _ in range(warmup):
            batch.launch(stream)
        if marks:
            region_mark()
        stream.synchronize()
        t0 = time.perf_counter()
        L.trn_event_record(events[0] if events else e0, stream.raw())
        for i in range(steps):
            batch.launch(stream)
            if events and i + 1 < steps:
                L.trn_event_record(events[i + 1], stream.raw())
        L.trn_event_record(events[steps] if events else e1, stream.raw())
        stream.synchronize()
        wall = (time.perf_counter() - t0) * 1e3
        if marks:
            region_mark()
            stream.synchronize()
        first, last = (events[0], events[steps]) if events else (e0, e1)
        return wall / steps, elapsed_ms(first, last) / steps

    # ---- timed region: W warm-up passes, then exactly K passes ------------------------------------------------
    ms_per_step, gpu_ms_per_step = run_passes(args.steps, args.warmup, events=pass_events, marks=True)
    value = total_bytes / (ms_per_step * 1e-3) / 1e9
    in_order = [round(elapsed_ms(pass_events[i], pass_events[i + 1]) * 1e3, 1) for i in range(args.steps)]
    per_pass = sorted(in_order)
    per_pass_us = {"min": per_pass[0], "median": per_pass[len(per_pass) // 2], "max": per_pass[-1], "in_order": in_order}

    # ---- what the timed passes left behind, against fp64 on the actual inputs: the last layer and the logits ------
    def norm64(v, eps=1e-6):
        v = v.astype(np.float64)
        return v / np.sqrt(np.mean(v * v) + eps)

    got = {nm: b.copy_to_host() for nm, b in dp.act_of_layer[layers - 1].items()}
    got["logits"] = logits.copy_to_host()
    x_last = xs[layers - 1].astype(np.float64)
    inputs = {"q": x_last, "k": x_last, "v": x_last, "gate": x_last, "up": x_last, "o": norm64(got["q"]), "down": norm64(got["gate"])}
    verification = {}
    for name, fmt, n, k in LAYER_MATS:
        w = kq.dequant_matrix(fmt, host_last[name], n, k)
        verification[f"layer{layers - 1}_{name}"] = float(kq.rel_l2(got[name], w @ inputs[name]))
        del w
    verification["head"] = float(kq.rel_l2(got["logits"], kq.dequant_matrix(HEAD[1], host_head, HEAD[2], HEAD[3]) @ norm64(got["down"])))
    worst = max(verification.values())
    assert np.all(np.isfinite(got["logits"])) and worst <= TOL, f"the timed pass is wrong: {verification}"
    del host_last, host_head

    # ---- dominant kernel: kq_gemv_many.  The library puts entries that are independent of one another (and of what
    #      they would overtake) into one launch; trn_kquant_gemv_plan says which entry of the pass goes into which.  A
    #      launch of more than sixteen entries runs kq_gemv_many: on this pass the first two launches, 97 % of the bytes.
    #      Second region: the same W + K passes, each pass issued as its launches one list each, in order, with an event
    #      between them on the stream.
    launch_of = batch.plan()
    members = {}
    for i, l in enumerate(launch_of):
        members.setdefault(l, []).append(i)
    lists, dominant = [], []
    for l in sorted(members):
        names = [entry_names[i] for i in members[l]]
        kinds = sorted(set(names), key=names.index)
        nbytes = sum(entry_bytes[i] for i in members[l])
        print(f"[bench] launch {l}: {len(names)} entries ({', '.join(f'{names.count(k)} x {k}' for k in kinds)}), {nbytes / 1e6:.1f} MB",
              file=sys.stderr, flush=True)
        g = batch.subset(members[l])
        assert len(set(g.plan())) == 1, "a launch of the pass, issued alone, must again be one launch"
        lists.append((g, nbytes, len(names) > 16))
    n_dom = sum(1 for _, _, dom in lists if dom)
    assert n_dom >= 1, "the pass has no launch of more than sixteen entries: the roofline section needs rewriting"
    dom_bytes = sum(nb for _, nb, dom in lists if dom)
    evs = [[ev() for _ in range(len(lists) + 1)] for _ in range(args.steps)]
    for _ in range(args.warmup):
        for g, _, _ in lists:
            g.launch(stream)
    region_mark()
    stream.synchronize()
    for p in range(args.steps):
        L.trn_event_record(evs[p][0], stream.raw())
        for j, (g, _, _) in enumerate(lists):
            g.launch(stream)
            L.trn_event_record(evs[p][j + 1], stream.raw())
    stream.synchronize()
    region_mark()
    stream.synchronize()
    dom_us = sum(elapsed_ms(evs[p][j], evs[p][j + 1]) * 1e3 for p in range(args.steps) for j, (_, _, dom) in enumerate(lists) if dom)
    grp_ms = dom_us / (n_dom * args.steps) * 1e-3
    region2_us_per_pass = elapsed_ms(evs[0][0], evs[-1][-1]) * 1e3 / args.steps
    per_launch_us = [round(sum(elapsed_ms(evs[p][j], evs[p][j + 1]) for p in range(args.steps)) * 1e3 / args.steps, 2) for j in range(len(lists))]
    n_grp = n_dom
    grp_bytes_per_launch = dom_bytes / n_dom
    achieved = grp_bytes_per_launch / (grp_ms * 1e-3) / 1e9

    # a bare read of as many bytes per launch, nothing computed (non-temporal 16-byte loads, every line once), launches
    # back to back over cold data: what the memory system and a kernel launch allow for a launch of this size
    read_bytes = int(grp_bytes_per_launch) // 16 * 16
    read_src = t.GpuBuffer(ctx, (2 * read_bytes + 4) // 4, np.float32)
    read_us = []
    for _ in range(5):
        L.trn_event_record(e0, stream.raw())
        for r in range(8):
            L.trn_read_u128(stream.raw(), read_src.as_ptr() + (r % 2) * read_bytes, read_bytes, y[4096].as_ptr())
        L.trn_event_record(e1, stream.raw())
        stream.synchronize()
        read_us.append(elapsed_ms(e0, e1) * 1e3 / 8)
    read_us = sorted(read_us)[2]
    read_src.free()

    traffic = None
    if os.path.exists(TRAFFIC_JSON):
        with open(TRAFFIC_JSON) as f:
            traffic = json.load(f)

    # ---- the same GEMVs wired as the strictly serial chain of a decoder ------------------------------------
    strict_ms = layer_ms = None
    if not args.pass_only:
        strict_ms, _ = run_passes(max(3, args.steps // 2), 2, strict_batch)
        layer_ms, _ = run_passes(max(3, args.steps // 2), 2, layer_batch)

    # ---- the same pass with ONE set of activation buffers shared by all layers, as a decoder's are: the write-after-
    #      read hazards between layers cut it into more, smaller launches.  Same logits, bit for bit. ----------------
    shared = None
    if not args.pass_only:
        shared_ms, _ = run_passes(max(3, args.steps // 2), 2, shared_batch)
        assert np.array_equal(logits.copy_to_host().view(np.uint32), got["logits"].view(np.uint32)), \
            "the pass with shared activation buffers must give the headline pass's logits"
        shared = {"us_per_pass": round(shared_ms * 1e3, 1), "gbps": round(total_bytes / shared_ms / 1e6, 1),
                  "frac_of_hbm_peak": round(total_bytes / shared_ms / 1e6 / HBM_PEAK_GBPS, 4), "launches": max(shared_batch.plan()) + 1}

    # ---- the same list through the one-launch executor (opt-in), for comparison ------------------------
    other_modes = {}
    if args.executors:
        L.trn_set_tuning(b"batch_mode", 1)
        ms, _ = run_passes(max(3, args.steps // 2), 1)
        other_modes["resident_phases"] = round(ms * 1e3, 1)
        L.trn_set_tuning(b"batch_mode", 0)

    # ---- timing protocol of the other configurations: launches back to back on the stream, no host wait inside;
    #      20 to warm up, then 5 batches of 200, the median batch counts.  "cold": every launch another of enough
    #      distinct device copies to make 1 GiB (nothing comes from the 256 MB last-level cache); "hot": one copy over
    #      and over; "grouped": eight copies per library call, which the library issues as one launch.
    def protocol(launch, reps=200, warm=20, batches=5):
        # a 4 KB read in front: in a kernel trace it separates this configuration's launches from the last one's
        L.trn_read_u128(stream.raw(), mark.as_ptr(), 4096, mark.as_ptr() + 4096)
        for r in range(warm):
            launch(r)
        stream.synchronize()
        us, enq = [], []
        for _ in range(batches):
            t0 = time.perf_counter()
            L.trn_event_record(e0, stream.raw())
            for r in range(reps):
                launch(r)
            L.trn_event_record(e1, stream.raw())
            enq.append((time.perf_counter() - t0) * 1e6 / reps)
            stream.synchronize()
            us.append(elapsed_ms(e0, e1) * 1e3 / reps)
        return sorted(us)[batches // 2], sorted(enq)[batches // 2]

    def copies_of(host, nbytes):
        n = max(2, -(-GIB // nbytes))
        first = t.GpuBuffer.from_host(ctx, host)
        bufs = [first]
        for _ in range(n - 1):
            b = t.GpuBuffer(ctx, first.len(), np.uint8)
            b.copy_from_buffer(first)
            bufs.append(b)
        return bufs

    def rate(nbytes, us):
        return {"us": round(us, 2), "gbps": round(nbytes / us / 1e3, 1), "frac_of_peak": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)}

    configs = {}
    if not args.no_configs:
        for label, fmt, n, k in (("1_q4k_gemv", "q4k", 4096, 4096), ("2_q6k_gemv", "q6k", 4096, 4096),
                                 ("2_q6k_gemv", "q6k", 32000, 4096), ("3_q5k_gemv", "q5k", 11008, 4096),
                                 ("3_q5k_gemv", "q5k", 4096, 11008), ("4_q4k_gemv", "q4k", 11008, 4096),
                                 ("4_q6k_gemv", "q6k", 4096, 11008)):
            nbytes = alg_bytes(fmt, n, k)
            bufs = copies_of(kq.gen_matrix(fmt, 1234, n, k), nbytes)
            nc = len(bufs)
            xb = x11008 if k == 11008 else dp.xs[0]
            fn = getattr(L, f"trn_{fmt}_gemv")
            cold, enq = protocol(lambda r: fn(stream.raw(), y[n].as_ptr(), bufs[r % nc].as_ptr(), xb.as_ptr(), k, n))
            hot, _ = protocol(lambda r: fn(stream.raw(), y[n].as_ptr(), bufs[0].as_ptr(), xb.as_ptr(), k, n))
            ys8 = [t.GpuBuffer(ctx, n, np.float32) for _ in range(8)]
            lists = []
            for c0 in range(0, nc - nc % 8 if nc >= 8 else nc, 8):
                b = t.GemvBatch()
                for j in range(8):
                    b.add(fmt, k, n, ys8[j], bufs[(c0 + j) % nc], xb)
                assert len(set(b.plan())) == 1
                lists.append(b)
            grouped, _ = protocol(lambda r: lists[r % len(lists)].launch(stream), reps=25, warm=4)
            row = {"cold": rate(nbytes, cold), "hot_last_level_cache": rate(nbytes, hot),
                   "grouped_8_per_call_cold": rate(nbytes, grouped / 8), "copies": nc, "host_enqueue_us_per_launch": round(enq, 2)}
            configs[f"{label}_{n}x{k}"] = row
            for b in bufs + ys8:
                b.free()
        for n, k in ((14336, 4096), (4096, 14336)):
            wbytes = n * (k // 256) * 144
            bufs = copies_of(kq.gen_matrix("q4k", 1238, n, k), wbytes)
            nc = len(bufs)
            for m in (1, 4, 16, 64):
                a = t.GpuBuffer.from_host(ctx, kq.gen_x(4321, m, k).reshape(-1))
                c = t.GpuBuffer(ctx, m * n, np.float32)
                cold, enq = protocol(lambda r: L.trn_q4k_gemm(stream.raw(), a.as_ptr(), bufs[r % nc].as_ptr(), c.as_ptr(), m, n, k))
                hot, _ = protocol(lambda r: L.trn_q4k_gemm(stream.raw(), a.as_ptr(), bufs[0].as_ptr(), c.as_ptr(), m, n, k))
                nbytes = wbytes + 4 * m * k + 4 * m * n
                row = {"cold": rate(nbytes, cold), "hot_last_level_cache": rate(nbytes, hot), "tflops": round(2.0 * m * n * k / cold / 1e6, 1),
                       "copies": nc, "host_enqueue_us_per_launch": round(enq, 2)}
                configs[f"5_q4k_gemm_{n}x{k}_m{m}"] = row
                a.free()
                c.free()
            for b in bufs:
                b.free()

        # the GEMM entry points outside the benchmark's named configurations: Q5_K / Q6_K and the legacy 18-byte format of
        # q4k_gemm_fused, 4096 x 4096
        n = k = 4096
        for fmt in ("q5k", "q6k"):
            bufs = copies_of(kq.gen_matrix(fmt, 1239, n, k), n * (k // 256) * SB[fmt])
            nc = len(bufs)
            fn = getattr(L, f"trn_{fmt}_gemm")
            for m in (4, 16, 64):
                a = t.GpuBuffer.from_host(ctx, kq.gen_x(4321, m, k).reshape(-1))
                c = t.GpuBuffer(ctx, m * n, np.float32)
                cold, _ = protocol(lambda r: fn(stream.raw(), a.as_ptr(), bufs[r % nc].as_ptr(), c.as_ptr(), m, n, k), reps=100, warm=8)
                configs[f"x_{fmt}_gemm_{n}x{k}_m{m}"] = {"cold": rate(alg_bytes(fmt, n, k) + 4 * (m - 1) * (k + n), cold), "copies": nc}
                a.free()
                c.free()
            for b in bufs:
                b.free()
        bufs = copies_of(kq.gen_q4k_simplified(np.random.default_rng(1240), n * (k // 32)), n * (k // 32) * 18)
        nc = len(bufs)
        for m in (1, 4):
            a = t.GpuBuffer.from_host(ctx, kq.gen_x(4321, m, k).reshape(-1))
            c = t.GpuBuffer(ctx, m * n, np.float32)
            cold, _ = protocol(lambda r: L.trn_q4k_gemm_fused(stream.raw(), a.as_ptr(), bufs[r % nc].as_ptr(), c.as_ptr(), m, n, k), reps=100, warm=8)
            configs[f"x_q4k_gemm_fused_{n}x{k}_m{m}"] = {"cold": rate(n * (k // 32) * 18 + 4 * m * (k + n), cold), "copies": nc}
            a.free()
            c.free()
        for b in bufs:
            b.free()

    # ---- the element-wise steps between the GEMVs of a layer, one launch each (latency-bound: a few KB) ----------
    glue_us = {}
    if not args.no_configs:
        hid, ffn = 4096, 11008
        g_a, g_b, g_o, g_g = (t.GpuBuffer.from_host(ctx, kq.gen_x(9000 + i, ffn)) for i in range(4))
        for label, fn in (("residual_add_4096", lambda r: L.trn_residual_add(stream.raw(), g_a.as_ptr(), g_b.as_ptr(), g_o.as_ptr(), hid)),
                          ("rmsnorm_4096", lambda r: L.trn_rmsnorm(stream.raw(), g_a.as_ptr(), g_o.as_ptr(), g_g.as_ptr(), hid, C.c_float(1e-5))),
                          ("fused_residual_rmsnorm_4096", lambda r: L.trn_fused_residual_rmsnorm(
                              stream.raw(), g_a.as_ptr(), g_b.as_ptr(), g_o.as_ptr(), g_g.as_ptr(), hid, C.c_float(1e-5))),
                          ("fused_swiglu_11008", lambda r: L.trn_fused_swiglu(stream.raw(), g_a.as_ptr(), g_b.as_ptr(), g_o.as_ptr(), ffn))):
            us, _ = protocol(fn, reps=100, warm=8)
            glue_us[label] = round(us, 2)

    # ---- the f32 GEMV of gemv.rs (A is K x N row-major) ---------------------------------------------------------
    f32_gemv = {}
    if not args.no_configs:
        rng = np.random.default_rng(55)
        for k, n in ((4096, 4096), (4096, 11008)):
            nbytes = 4 * k * n + 4 * k + 4 * n
            bufs = copies_of(rng.standard_normal(k * n, dtype=np.float32).view(np.uint8), nbytes)
            nc = len(bufs)
            xb, yb = dp.xs[0], y[n]
            cold, _ = protocol(lambda r: L.trn_gemv_f32(stream.raw(), yb.as_ptr(), bufs[r % nc].as_ptr(), xb.as_ptr(), k, n), reps=100, warm=8)
            f32_gemv[f"k{k}_n{n}"] = {"cold": rate(nbytes, cold), "copies": nc}
            for b in bufs:
                b.free()

    # ---- single-query attention over a KV cache of 7B shape (32 heads x 128) -----------------------------------
    attention = {}
    if not args.no_configs:
        rng = np.random.default_rng(66)
        heads, dim = 32, 128
        for seq in (512, 2048, 8192):
            nbytes = 8 * heads * seq * dim + 8 * heads * dim
            host = rng.standard_normal(heads * seq * dim, dtype=np.float32).view(np.uint8)
            kb, vb = copies_of(host, nbytes // 2), copies_of(host, nbytes // 2)
            nc = len(kb)
            qb, ob = dp.xs[0], y[4096]
            cold, _ = protocol(lambda r: L.trn_incremental_attention(stream.raw(), qb.as_ptr(), kb[r % nc].as_ptr(), vb[r % nc].as_ptr(),
                                                                     ob.as_ptr(), seq, dim, heads, heads, seq, C.c_float(dim ** -0.5)),
                               reps=100, warm=8)
            attention[f"seq{seq}"] = {"cold": rate(nbytes, cold), "copies": nc}
            for b in kb + vb:
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
    cpu_configs = None
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
        cpu_configs = {"1_q4k_4096x4096": {"cores": cores, "dequant_matvec_us": round(sec_dq / 5 * 1e6, 1),
                                           "dequant_matvec_gbps_quantized": round(alg_bytes("q4k", n1, k1) / (sec_dq / 5) / 1e9, 2),
                                           "matvec_predequantised_f32_us": round(sec_mv / 5 * 1e6, 1),
                                           "matvec_predequantised_gbps_quantized": round(alg_bytes("q4k", n1, k1) / (sec_mv / 5) / 1e9, 2)}}
        # configurations 2 and 3 on the CPU path (dequantise + matvec per call)
        for label, fmt, n, k in (("2_q6k_4096x4096", "q6k", 4096, 4096), ("2_q6k_32000x4096", "q6k", 32000, 4096),
                                 ("3_q5k_11008x4096", "q5k", 11008, 4096), ("3_q5k_4096x11008", "q5k", 4096, 11008)):
            wm = kq.gen_matrix(fmt, 1234 + n + k, n, k)
            _, sec = cb.dequant_matvec(fmt, wm, hx[k], k, n, cores, 3)
            cpu_configs[label] = {"dequant_matvec_us": round(sec / 3 * 1e6, 1),
                                  "dequant_matvec_gbps_quantized": round(alg_bytes(fmt, n, k) / (sec / 3) / 1e9, 2)}
        cpu = {"value": round(layer_bytes * reps / spent / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"layer 0 of the pass (7 GEMVs, {layer_bytes / 1e6:.1f} MB quantized) x {reps} repetitions, "
                         f"dequantise-row + AVX2 dot, {'AVX2+FMA' if cb.has_avx2() else 'scalar'}"}

    def chain(ms):
        if ms is None:
            return None
        return {"us_per_pass": round(ms * 1e3, 1), "gbps": round(total_bytes / ms / 1e6, 1),
                "frac_of_hbm_peak": round(total_bytes / ms / 1e6 / HBM_PEAK_GBPS, 4)}

    out = {
        "metric": "k-quant GEMV achieved HBM GB/s (% of peak) + µs per 7B decode weight pass",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"7B-style decode weight pass: {layers} layers x (4x Q4_K 4096x4096 + 2x Q4_K 11008x4096 + "
                               f"1x Q6_K 4096x11008) + Q6_K 32000x4096 head; {len(batch)} GEMVs in layer order "
                               f"(per layer x_l~N(0,1) -> q,k,v,gate,up; o<-norm(q); down<-norm(gate); head<-norm(down); "
                               f"activation buffers per layer), "
                               f"{total_bytes / 1e9:.3f} GB, batch 1, f32 x and y", "gemvs": len(batch),
                   "bytes_per_step": total_bytes, "launches_per_step": max(launch_of) + 1,
                   # the same matrices in the data flow of a real decoder: every step waits for the one before it
                   "strict_decoder_chain": chain(strict_ms) and dict(chain(strict_ms), dependent_steps=max(strict_batch.plan()) + 1),
                   "strict_decoder_chain_with_folded_layer_glue": chain(layer_ms),
                   # the headline's data flow with one set of activation buffers for all layers (more, smaller launches)
                   "same_pass_with_shared_activation_buffers": shared},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "traffic": traffic["bytes_per_launch"] if traffic else None,
                     "traffic_measured_at": traffic.get("commit") if traffic else None,
                     "kernel": "kq_gemv_many", "launches_per_pass": n_grp,
                     "bytes_per_launch": round(grp_bytes_per_launch), "us_per_launch": round(grp_ms * 1e3, 3),
                     # the region these launches were timed in: every launch of a pass as a list of its own, events between
                     "us_per_pass_in_this_region": round(region2_us_per_pass, 1), "us_per_launch_of_the_pass_in_order": per_launch_us,
                     # the whole pass of the headline region against the peak (head, launch gaps and all): a lower bound
                     "frac_of_peak_from_ms_per_step": round(value / HBM_PEAK_GBPS, 4),
                     # a launch that only reads as many bytes (trn_read_u128), same protocol: the ceiling for a launch of this size
                     "bare_read_us_per_launch": round(read_us, 3), "bare_read_gbps": round(read_bytes / read_us / 1e3, 1),
                     "frac_of_bare_read": round(read_us / (grp_ms * 1e3), 4)},
        "cpu_baseline": cpu,
        "extra": {"us_per_pass": round(ms_per_step * 1e3, 1), "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
                  "gpu_event_us_per_pass": round(gpu_ms_per_step * 1e3, 1), "per_pass_us": per_pass_us,
                  "verification_after_timed_region_rel_l2_vs_fp64": dict(verification, tolerance=TOL),
                  "us_per_pass_strict_decoder_chain": strict_ms and round(strict_ms * 1e3, 1),
                  "us_per_pass_one_launch_executors": other_modes,
                  "weight_bytes": weight_bytes, "us_per_pass_decoder_chain_with_folded_layer_glue": layer_ms and round(layer_ms * 1e3, 1),
                  "configs_200_launches_median_of_5": configs,
                  "layer_glue_us_per_launch_back_to_back": glue_us, "decode_step_7b_folded_glue_and_attention": decode_step,
                  "f32_gemv": f32_gemv, "incremental_attention_32x128": attention,
                  "cpu_configs": cpu_configs, "device": ctx.device_name(), "cus": ctx.cu_count()},
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
