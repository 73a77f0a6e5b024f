"""The f32 GEMV kernels of gemv.rs (gemv_warp_reduce, gemv_coalesced): y[n] = sum_k A[k][n] x[k] with A K x N row-major.
Oracle pins on the CPU; parity of the GPU kernel through the C ABI to 1e-5 relative L2 against fp64 and no worse than
1.5x the f32 evaluations in the reference's two summation orders."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import glue
from oracle import kquant as kq

TOL = 1e-5


def test_names_and_geometry_follow_the_reference():
    assert t.GemvKernel(4096, 32000).name() == "gemv_warp_reduce"            # gemv.rs:41-43
    assert t.CoalescedGemvKernel(4096, 4096).name() == "gemv_coalesced"      # :208-210
    assert t.GemvKernel(64, 100).launch_config().grid == (100, 1, 1)         # one warp per output element
    assert t.GemvKernel(64, 100).launch_config().block == (32, 1, 1)
    c = t.CoalescedGemvKernel(64, 1000).launch_config()
    assert c.grid == (4, 1, 1) and c.block == (256, 1, 1) and c.shared_mem == 1024      # :217-227


def test_oracle_orders_on_a_tiny_case_by_brute_force():
    rng = np.random.default_rng(1)
    k, n = 70, 5
    a, x = rng.standard_normal((k, n)).astype(np.float32), rng.standard_normal(k).astype(np.float32)
    want = np.array([sum(float(a[i, j]) * float(x[i]) for i in range(k)) for j in range(n)])
    assert np.allclose(glue.gemv_f32_fp64(a, x), want, rtol=1e-14)
    for f in (glue.gemv_f32_coalesced_order, glue.gemv_f32_warp_reduce_order):
        assert kq.rel_l2(f(a, x), want) <= 3e-7
    # A is K x N: a one-hot x picks a ROW of A
    e = np.zeros(k, np.float32)
    e[13] = 2.0
    assert np.array_equal(glue.gemv_f32_coalesced_order(a, e), 2.0 * a[13])
    assert np.array_equal(glue.gemv_f32_warp_reduce_order(a, e), 2.0 * a[13])


@pytest.mark.gpu
@pytest.mark.parametrize("k,n", [(4096, 4096), (1000, 1028), (64, 256), (7, 4), (3000, 999), (512, 6), (1, 260), (11008, 512)])
def test_gpu_gemv_f32(gpu, k, n):
    ctx, stream = gpu
    rng = np.random.default_rng(k * 31 + n)
    a, x = rng.standard_normal((k, n)).astype(np.float32), rng.standard_normal(k).astype(np.float32)
    da, dx = t.GpuBuffer.from_host(ctx, a.reshape(-1)), t.GpuBuffer.from_host(ctx, x)
    dy = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
    t.GemvKernel(k, n).launch(stream, dy, da, dx)
    stream.synchronize()
    got, want = dy.copy_to_host(), glue.gemv_f32_fp64(a, x)
    err = kq.rel_l2(got, want)
    assert err <= TOL, err
    if n >= 256 and k >= 256 and k * n <= 1100 * 1100:      # enough outputs and terms for the ratio of two errors to mean something
        ref = max(kq.rel_l2(glue.gemv_f32_coalesced_order(a, x), want), kq.rel_l2(glue.gemv_f32_warp_reduce_order(a, x), want))
        assert err <= 1.5 * ref + 1e-9, (err, ref)
    again = t.GpuBuffer.from_host(ctx, np.zeros(n, np.float32))
    t.CoalescedGemvKernel(k, n).launch(stream, again, da, dx)          # the same engine under the other name
    stream.synchronize()
    assert np.array_equal(again.copy_to_host().view(np.uint32), got.view(np.uint32))


@pytest.mark.gpu
def test_gpu_gemv_f32_by_name_and_edges(gpu):
    ctx, stream = gpu
    module = t.CudaModule.from_builtin(ctx)
    k, n = 300, 520
    rng = np.random.default_rng(9)
    a, x = rng.standard_normal((k, n)).astype(np.float32), rng.standard_normal(k).astype(np.float32)
    da, dx = t.GpuBuffer.from_host(ctx, a.reshape(-1)), t.GpuBuffer.from_host(ctx, x)
    want = glue.gemv_f32_fp64(a, x)
    for K in (t.GemvKernel, t.CoalescedGemvKernel):
        dy = t.GpuBuffer.from_host(ctx, np.zeros(n, np.float32))
        K(k, n).launch_by_name(stream, module, dy, da, dx)
        stream.synchronize()
        assert kq.rel_l2(dy.copy_to_host(), want) <= TOL
    L = t._ffi.lib()
    dy = t.GpuBuffer.from_host(ctx, np.full(8, 5.0, np.float32))
    assert L.trn_gemv_f32(stream.raw(), dy.as_ptr(), da.as_ptr(), dx.as_ptr(), k, 0) == 0        # n = 0
    assert L.trn_gemv_f32(stream.raw(), dy.as_ptr(), da.as_ptr(), dx.as_ptr(), 0, 8) == 0        # k = 0: y = 0
    stream.synchronize()
    assert np.all(dy.copy_to_host() == 0.0)
    assert L.trn_gemv_f32(stream.raw(), 0, da.as_ptr(), dx.as_ptr(), k, n) != 0
