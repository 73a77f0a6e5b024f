"""GPU tests of the drop-in boundary's corners: the built-in image loaded through trn_module_load_data, kernels that
are not reference names, by-name launches with exactly the reference's parameter lists (layernorm.rs:426-428,
elementwise.rs:146-149, attention.rs:897-901), and two host threads on two streams."""
import ctypes as C
import threading

import numpy as np
import pytest

import trueno_amd as t
from oracle import glue as og
from oracle import kquant as kq
from trueno_amd import _ffi

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _builtin_bytes():
    L = _ffi.lib()
    img, size = C.c_void_p(), C.c_size_t()
    assert L.trn_builtin_image(C.byref(img), C.byref(size)) == 0
    return C.string_at(img.value, size.value)


def test_builtin_image_through_load_data_keeps_the_kernels_geometry(gpu):
    """the reference's geometry (grid = N blocks of 32 threads, no shared memory) must not reach the engine raw"""
    ctx, stream = gpu
    mod = t.CudaModule.from_image(ctx, _builtin_bytes())          # a COPY of the image, not the library's own pointer
    n, k = 300, 1024
    for fmt, kern in (("q4k", t.Q4KGemvKernel), ("q5k", t.Q5KGemvKernel), ("q6k", t.Q6KGemvKernel)):
        buf, x = kq.gen_matrix(fmt, 3, n, k), kq.gen_x(4, k)
        dw, dx = t.GpuBuffer.from_host(ctx, buf), t.GpuBuffer.from_host(ctx, x)
        dy = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
        kk = kern(k, n)
        assert kk.launch_config().block == (32, 1, 1)
        kk.launch_by_name(stream, mod, dy, dw, dx)
        stream.synchronize()
        assert kq.rel_l2(dy.copy_to_host(), kq.gemv_fp64(kq.dequant_matrix(fmt, buf, n, k), x)) <= TOL, fmt


def test_internal_kernels_are_not_launchable_by_name(gpu):
    ctx, stream = gpu
    for mod in (t.CudaModule.from_builtin(ctx), t.CudaModule.from_image(ctx, _builtin_bytes())):
        for name in ("kq_gemv_group", "q4k_gemv_flags", "kq_gemv_phases", "q4k_gemm_f16_w8"):
            with pytest.raises(t.GpuError) as e:
                stream.launch_kernel(mod, name, t.LaunchConfig((4, 1, 1), (32, 1, 1), 0), [C.c_uint64(0)] * 12)
            assert e.value.kind == "KernelLaunch" and e.value.code == 1, name
    stream.synchronize()


def test_norm_and_attention_by_name_take_only_the_reference_parameters(gpu):
    ctx, stream = gpu
    L = _ffi.lib()
    hidden = 1024
    x, g, r = kq.gen_x(5, hidden), kq.gen_x(6, hidden), kq.gen_x(7, hidden)
    dx, dg, dr = (t.GpuBuffer.from_host(ctx, v) for v in (x, g, r))
    do = t.GpuBuffer.from_host(ctx, np.full(hidden, np.nan, np.float32))
    mod = t.CudaModule.from_builtin(ctx)
    # without the instance constants the launch is refused (and reads nothing beyond the three pointers)
    three = [C.c_uint64(dx.as_ptr()), C.c_uint64(do.as_ptr()), C.c_uint64(dg.as_ptr())]
    with pytest.raises(t.GpuError) as e:
        stream.launch_kernel(mod, "rmsnorm", t.LaunchConfig((1, 1, 1), (32, 1, 1), 0), three)
    assert e.value.code == 1
    kern = t.RmsNormKernel(hidden).with_epsilon(1e-6)
    assert len(kern.kernel_args(dx, do, dg)) == 3
    kern.launch_by_name(stream, mod, dx, do, dg)
    stream.synchronize()
    assert kq.rel_l2(do.copy_to_host(), og.rmsnorm_fp64(x, g, 1e-6)) <= TOL
    mod2 = t.CudaModule.from_builtin(ctx)
    k2 = t.FusedResidualRmsNormKernel(hidden)
    assert len(k2.kernel_args(dr, dx, do, dg)) == 4
    k2.launch_by_name(stream, mod2, dr, dx, do, dg)
    stream.synchronize()
    assert kq.rel_l2(do.copy_to_host(), og.rmsnorm_fp64((r + x).astype(np.float32), g, 1e-5)) <= TOL
    # the setters only take the kernels they belong to
    assert L.trn_function_set_rmsnorm(mod.get_function("residual_add"), hidden, 1e-5) == 1
    assert L.trn_function_set_attention(mod.get_function("rmsnorm"), 64, 1, 1, 16, 0.125) == 1
    with pytest.raises(t.GpuError):
        stream.launch_kernel(t.CudaModule.from_builtin(ctx), "incremental_attention",
                             t.LaunchConfig((1, 1, 1), (32, 1, 1), 0), [C.c_uint64(dx.as_ptr())] * 4 + [C.c_uint32(1)])
    stream.synchronize()


def test_two_threads_two_streams(gpu):
    """workspaces are per (device, stream) and grown under a lock: two host threads, each with its own stream, issue
    GEMMs (matrix-core form, K cut in parts -> scratch buffer), f32 GEMVs and attention concurrently"""
    ctx, _ = gpu
    n, k = 1024, 2048
    buf = kq.gen_matrix("q4k", 11, n, k)
    w = kq.dequant_matrix("q4k", buf, n, k)
    dw = t.GpuBuffer.from_host(ctx, buf)
    results, errors = {}, []

    def worker(tid):
        try:
            ctx.make_current()
            stream = t.CudaStream(ctx)
            outs = []
            for rep in range(6):
                m = 4 + 12 * ((rep + tid) % 3)            # different sizes: the scratch buffer grows
                a = kq.gen_x(100 + 10 * tid + rep, m, k)
                da = t.GpuBuffer.from_host(ctx, a)
                dc = t.GpuBuffer.from_host(ctx, np.full(m * n, np.nan, np.float32))
                t.QuantizeKernel.ggml(m, n, k).launch(stream, da, dw, dc)
                stream.synchronize()
                outs.append((a, dc.copy_to_host().reshape(m, n)))
            stream.destroy()
            results[tid] = outs
        except Exception as exc:      # noqa: BLE001 - reported below
            errors.append((tid, repr(exc)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
    for tid, outs in results.items():
        for a, c in outs:
            assert kq.rel_l2(c, kq.gemm_fp64(a, w)) <= TOL, tid
