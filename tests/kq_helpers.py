"""Shared helpers for the GPU parity tests: upload, launch through the C ABI, download."""
from __future__ import annotations

import json
import os
import tempfile

import numpy as np

import trueno_amd as t
from trueno_amd import kernels as K

GEMV_KERNEL = {"q4k": t.Q4KGemvKernel, "q5k": t.Q5KGemvKernel, "q6k": t.Q6KGemvKernel}
GEMM_KERNEL = {"q4k": t.QuantizeKernel.ggml, "q5k": t.Q5KKernel, "q6k": t.Q6KKernel}
SB = {"q4k": 144, "q5k": 176, "q6k": 210}

# Our error against fp64 may be at most this multiple of the error of an f32 evaluation in the reference's own
# summation order (trueno-gpu/src/kernels/quantize.rs:1412, 1482-1518).  The clause is "no worse than": 1.0, plus a
# sampling margin - both errors are sums over a few thousand rounding errors, so their ratio scatters by about
# 1 / sqrt(rows) around its expectation (1.6 % with 4096 rows, 2.2 % with 2048, 3.1 % with 1024).
REF_SLACK = 1.05
# where the ratios go: a file named by TRN_RATIO_LOG, else one in the temporary directory
RATIO_LOG = os.environ.get("TRN_RATIO_LOG") or os.path.join(tempfile.gettempdir(), "trueno_ref_order_ratios.jsonl")


def record_ratio(kind: str, fmt: str, m: int, n: int, k: int, rows: int, ours: float, ref: float) -> None:
    """one line per measured shape: our relative L2 error against fp64 over the reference-order f32 evaluation's"""
    os.makedirs(os.path.dirname(RATIO_LOG), exist_ok=True)
    with open(RATIO_LOG, "a") as f:
        f.write(json.dumps({"kind": kind, "fmt": fmt, "m": m, "n": n, "k": k, "rows": rows, "ours": ours, "reference_order": ref,
                            "ratio": ours / ref if ref > 0 else None}) + "\n")


def gpu_dequant(gpu, fmt: str, buf: np.ndarray, policy: int = 0, w_offset: int = 0) -> np.ndarray:
    ctx, stream = gpu
    buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
    n_sb = buf.size // SB[fmt]
    dw = t.GpuBuffer(ctx, buf.size + w_offset, np.uint8)
    dw.copy_from_host_at(buf, w_offset)
    out = t.GpuBuffer(ctx, n_sb * 256, np.float32)
    K.dequant_f32(fmt, stream, out, dw.as_ptr() + w_offset, n_sb, policy)
    stream.synchronize()
    return out.copy_to_host().reshape(n_sb, 256)


def gpu_gemv(gpu, fmt: str, buf: np.ndarray, x: np.ndarray, k: int, n: int, *, by_name=None,
             w_offset: int = 0, x_offset: int = 0, fill: float = np.nan) -> np.ndarray:
    """y = W x on the GPU.  by_name: a CudaModule to go through launch_kernel with the reference's
    LaunchConfig instead of the typed launcher.  Offsets (bytes / elements) misalign the operands."""
    ctx, stream = gpu
    buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
    dw = t.GpuBuffer(ctx, buf.size + w_offset, np.uint8)
    dw.copy_from_host_at(buf, w_offset)
    dx = t.GpuBuffer(ctx, k + x_offset, np.float32)
    dx.copy_from_host_at(np.ascontiguousarray(x, np.float32), x_offset)
    dy = t.GpuBuffer.from_host(ctx, np.full(max(n, 1), fill, np.float32))
    kern = GEMV_KERNEL[fmt](k, n)
    wp, xp = dw.as_ptr() + w_offset, dx.as_ptr() + 4 * x_offset
    if by_name is not None:
        kern.launch_by_name(stream, by_name, dy, wp, xp)
    else:
        kern.launch(stream, dy, wp, xp)
    stream.synchronize()
    return dy.copy_to_host()[:n]


def gpu_gemm(gpu, fmt: str, buf: np.ndarray, a: np.ndarray, m: int, n: int, k: int, *, by_name=None, as_written=False) -> np.ndarray:
    ctx, stream = gpu
    dw = t.GpuBuffer.from_host(ctx, np.ascontiguousarray(buf, np.uint8).reshape(-1))
    da = t.GpuBuffer.from_host(ctx, np.ascontiguousarray(a, np.float32).reshape(-1))
    dc = t.GpuBuffer.from_host(ctx, np.full(max(m * n, 1), np.nan, np.float32))
    kern = GEMM_KERNEL[fmt](m, n, k)
    if by_name is not None:
        kern.launch_by_name(stream, by_name, da, dw, dc)
    else:
        kern.launch(stream, da, dw, dc, as_written)
    stream.synchronize()
    return dc.copy_to_host()[: m * n].reshape(m, n)
