"""GPU parity, batched GEMM C = A . dequant(W)^T: within 1e-5 relative L2 of fp64 for M in {1, 4, 16, 64},
row-major C, m = 1 equal to the GEMV; typed launcher and launch-by-name."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from tests.kq_helpers import gpu_gemm, gpu_gemv

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _c64(fmt, buf, a, n, k):
    return kq.gemm_fp64(a, kq.dequant_matrix(fmt, buf, n, k))


@pytest.mark.parametrize("m", (1, 4, 16, 64))
@pytest.mark.parametrize("fmt,n,k", [("q4k", 1024, 4096), ("q4k", 520, 14336), ("q5k", 300, 1024), ("q6k", 300, 2048)])
def test_gemm_against_fp64(gpu, fmt, n, k, m):
    buf, a = kq.gen_matrix(fmt, 200 + m, n, k), kq.gen_x(300 + m, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert c.shape == (m, n) and np.all(np.isfinite(c))
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL


@pytest.mark.parametrize("m", (1, 4, 16, 64))
def test_gemm_config_shape_w_14336x4096(gpu, m):
    n, k = 14336, 4096
    buf, a = kq.gen_matrix("q4k", 1234, n, k), kq.gen_x(4321, m, k)
    c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
    assert kq.rel_l2(c, _c64("q4k", buf, a, n, k)) <= TOL


def test_gemm_config_shape_w_4096x14336(gpu):
    n, k, m = 4096, 14336, 16
    buf, a = kq.gen_matrix("q4k", 1235, n, k), kq.gen_x(4322, m, k)
    c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
    assert kq.rel_l2(c, _c64("q4k", buf, a, n, k)) <= TOL


@pytest.mark.parametrize("fmt", ("q4k", "q5k", "q6k"))
def test_gemm_m1_equals_gemv_and_by_name(gpu, fmt):
    ctx, _ = gpu
    n, k = 777, 1536
    buf, a = kq.gen_matrix(fmt, 7, n, k), kq.gen_x(8, 3, k)
    y = gpu_gemv(gpu, fmt, buf, a[0], k, n)
    c1 = gpu_gemm(gpu, fmt, buf, a[:1], 1, n, k)
    assert kq.rel_l2(c1[0], y.astype(np.float64)) <= 2e-7
    mod = t.CudaModule.from_builtin(ctx)
    c3 = gpu_gemm(gpu, fmt, buf, a, 3, n, k, by_name=mod)
    assert kq.rel_l2(c3, _c64(fmt, buf, a, n, k)) <= TOL
    assert kq.rel_l2(c3[0], y.astype(np.float64)) <= 2e-7


def test_gemm_edge_cases(gpu):
    ctx, stream = gpu
    a = t.GpuBuffer.from_host(ctx, np.ones(256, np.float32))
    w = t.GpuBuffer.from_host(ctx, np.zeros(144, np.uint8))
    c = t.GpuBuffer.from_host(ctx, np.full(4, 3.0, np.float32))
    t.QuantizeKernel.ggml(0, 1, 256).launch(stream, a, w, c)      # m = 0: nothing written
    t.QuantizeKernel.ggml(1, 0, 256).launch(stream, a, w, c)      # n = 0
    stream.synchronize()
    assert np.all(c.copy_to_host() == 3.0)
    with pytest.raises(t.GpuError):
        t.QuantizeKernel.ggml(1, 1, 300).launch(stream, a, w, c)  # k % 256 != 0
