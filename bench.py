#!/usr/bin/env python3
"""Benchmark of the k-quant GEMV path on one MI355X.

A step is one 7B-style decode weight pass: 32 layers x {Q,K,V,O: Q4_K 4096x4096; gate, up: Q4_K
11008x4096; down: Q6_K 4096x11008} plus the Q6_K 32000x4096 head - 225 GEMVs over 4.12 GB of
distinct, seeded synthetic weights resident in HBM (far beyond the 256 MB Infinity Cache, so every
pass streams from HBM).  The GEMVs of a pass are issued in order on one stream; within a layer
Q, K, V, O, gate, up read the layer's activation vector x_l ~ N(0,1) (4096) and down reads a second
N(0,1) vector (11008).  `value` is algorithmic bytes (weights + x + y, each once) over wall time.

Prints one JSON line.  Extra fields: `roofline` for the dominant kernel (Q4_K GEMV: 2.83 of the
4.12 GB), timed per launch with HIP events on the launch stream; `cpu_baseline`: the CPU port
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
    ap.add_argument("--layers", type=int, default=LAYERS, help=argparse.SUPPRESS)
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this path runs on one GPU; --gpus must be 1 (a multi-GPU run would shard W by rows, "
              "see DESIGN.md)", file=sys.stderr)
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

    batch = t.GemvBatch()
    q4_batch = t.GemvBatch()
    total_bytes = q4_bytes = 0
    for layer in range(layers):
        x4096, x11008 = xs[layer]
        for name, fmt, n, k in LAYER_MATS:
            x = x11008 if k == 11008 else x4096
            batch.add(fmt, k, n, ys[name], weights[layer][name], x)
            total_bytes += alg_bytes(fmt, n, k)
            if fmt == "q4k":
                q4_batch.add(fmt, k, n, ys[name], weights[layer][name], x)
                q4_bytes += alg_bytes(fmt, n, k)
    batch.add(HEAD[1], HEAD[3], HEAD[2], y[32000], head_w, xs[-1][0])
    total_bytes += alg_bytes(HEAD[1], HEAD[2], HEAD[3])

    def ev():
        e = C.c_void_p()
        assert L.trn_event_create(C.byref(e)) == 0
        return e

    def elapsed_ms(a, b):
        ms = C.c_float()
        assert L.trn_event_elapsed_ms(C.byref(ms), a, b) == 0
        return float(ms.value)

    # ---- timed region: W warm-up passes, then exactly K passes ------------------------------------
    for _ in range(args.warmup):
        batch.launch(stream)
    stream.synchronize()
    e0, e1 = ev(), ev()
    t0 = time.perf_counter()
    L.trn_event_record(e0, stream.raw())
    for _ in range(args.steps):
        batch.launch(stream)
    L.trn_event_record(e1, stream.raw())
    stream.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = elapsed_ms(e0, e1)
    ms_per_step = wall_ms / args.steps
    value = total_bytes / (ms_per_step * 1e-3) / 1e9

    # ---- dominant kernel (Q4_K GEMV), per launch, HIP events on the launch stream ------------------
    n_q4 = len(q4_batch)
    evs = [ev() for _ in range(n_q4 + 1)]
    one = []
    for layer in range(layers):
        for name, fmt, n, k in LAYER_MATS:
            if fmt == "q4k":
                one.append(t.GemvBatch().add(fmt, k, n, ys[name], weights[layer][name], xs[layer][0]))
    durations = []
    for rep in range(3):
        stream.synchronize()
        L.trn_event_record(evs[0], stream.raw())
        for i, b in enumerate(one):
            b.launch(stream)
            L.trn_event_record(evs[i + 1], stream.raw())
        stream.synchronize()
        durations.append(sum(elapsed_ms(evs[i], evs[i + 1]) for i in range(n_q4)) / n_q4)
    q4_ms = min(durations)
    q4_bytes_per_launch = q4_bytes / n_q4
    achieved = q4_bytes_per_launch / (q4_ms * 1e-3) / 1e9

    # ---- per-shape steady-state table (cold: rotates through the 32 layers' copies) ----------------
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

    # ---- CPU baseline: the port, layer 0's seven matrices, all host cores --------------------------
    cpu = None
    if not args.no_cpu_baseline:
        from oracle.cref import CpuBaseline
        cb = CpuBaseline()
        # the GPU box gives this job a share of the host's cores; do not oversubscribe it
        cores = max(1, min(cb.threads(), int(os.environ.get("OMP_NUM_THREADS", cb.threads()))))
        hx = {4096: kq.gen_x(4321, 4096), 11008: kq.gen_x(8321, 11008)}
        layer_bytes = sum(alg_bytes(fmt, n, k) for _, fmt, n, k in LAYER_MATS)
        reps, spent = 0, 0.0
        t_start = time.time()
        while (spent < 10.0 and reps < 200) or reps < 2:
            for name, fmt, n, k in LAYER_MATS:
                _, sec = cb.dequant_matvec(fmt, host_layer0[name], hx[k], k, n, cores, 1)
                spent += sec
            reps += 1
            if time.time() - t_start > 40:
                break
        cpu = {"value": round(layer_bytes * reps / spent / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
               "sample": f"layer 0 of the pass (7 GEMVs, {layer_bytes / 1e6:.1f} MB quantized) x {reps} repetitions, "
                         f"dequantise-row + AVX2 dot, {'AVX2+FMA' if cb.has_avx2() else 'scalar'}"}

    out = {
        "metric": "k-quant GEMV achieved HBM GB/s over a 7B decode weight pass",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"7B-style decode weight pass: {layers} layers x (4x Q4_K 4096x4096 + 2x Q4_K 11008x4096 + "
                               f"1x Q6_K 4096x11008) + Q6_K 32000x4096 head; {len(batch)} GEMVs, {total_bytes / 1e9:.3f} GB, "
                               "batch 1, f32 x and y", "gemvs": len(batch), "bytes_per_step": total_bytes},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
                     "kernel": "q4k_gemv_warp_reduce", "launches": n_q4,
                     "bytes_per_launch": round(q4_bytes_per_launch), "us_per_launch": round(q4_ms * 1e3, 3)},
        "cpu_baseline": cpu,
        "extra": {"us_per_pass": round(ms_per_step * 1e3, 1), "frac_of_hbm_peak": round(value / HBM_PEAK_GBPS, 4),
                  "gpu_event_ms_per_step": round(gpu_ms / args.steps, 4), "per_shape_cold": shapes,
                  "device": ctx.device_name(), "cus": ctx.cu_count()},
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
