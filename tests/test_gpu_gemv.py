"""GPU parity, GEMV: y = W x within 1e-5 relative L2 of the fp64 product of the oracle-dequantised
weights, and no worse than an f32 evaluation in the reference's own summation order, at the
benchmark shapes and at the edge cases; through the typed launchers and through launch-by-name
with the reference's LaunchConfig."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import _ffi
from tests.kq_helpers import REF_SLACK, gpu_gemv, record_ratio

pytestmark = pytest.mark.gpu

TOL = 1e-5          # relative L2 against fp64 (the stated tolerance of the path)


def _check(gpu, coracle, fmt, n, k, seed, *, by_name=None, ref_rows=4096):
    buf = kq.gen_matrix(fmt, seed, n, k)
    x = kq.gen_x(seed + 1, k)
    y = gpu_gemv(gpu, fmt, buf, x, k, n, by_name=by_name)
    assert np.all(np.isfinite(y))
    y64 = np.empty(n, np.float64)
    step = 2048
    nsb = k // 256
    sb = kq.SB_BYTES[fmt]
    for r0 in range(0, n, step):
        r1 = min(n, r0 + step)
        w = kq.dequant_matrix(fmt, buf[r0 * nsb * sb:r1 * nsb * sb], r1 - r0, k)
        y64[r0:r1] = kq.gemv_fp64(w, x)
    err = kq.rel_l2(y, y64)
    assert err <= TOL, err
    # the reference's own f32 result, emulated on a row sample (a ratio of two rounding-noise
    # figures means nothing on a handful of rows)
    if n < 1024 or ref_rows < 1024:
        return err, None
    rows = min(n, ref_rows)
    yref = coracle.gemv_ref_order_f32(fmt, buf[: rows * nsb * sb], x, k, rows)
    err_ref = kq.rel_l2(yref, y64[:rows])
    err_ours = kq.rel_l2(y[:rows], y64[:rows])
    record_ratio("gemv", fmt, 1, n, k, rows, err_ours, err_ref)
    assert err_ours <= REF_SLACK * err_ref, (fmt, n, k, err_ours, err_ref, err_ours / err_ref)
    return err, err_ref


# the shapes the benchmark configurations name
@pytest.mark.parametrize("fmt,n,k", [
    ("q4k", 4096, 4096),
    ("q6k", 4096, 4096), ("q6k", 32000, 4096),
    ("q5k", 11008, 4096), ("q5k", 4096, 11008),
    ("q4k", 11008, 4096), ("q6k", 4096, 11008),
    ("q4k", 14336, 4096), ("q4k", 4096, 14336),
])
def test_gemv_config_shapes(gpu, coracle, fmt, n, k):
    _check(gpu, coracle, fmt, n, k, seed=1234)


@pytest.mark.parametrize("fmt", ("q4k", "q5k", "q6k"))
@pytest.mark.parametrize("n,k", [(1, 256), (3, 512), (5, 4096), (17, 4352), (63, 256), (257, 768), (1000, 8192),
                                 (33, 12544)])
def test_gemv_ragged_shapes(gpu, coracle, fmt, n, k):
    _check(gpu, coracle, fmt, n, k, seed=77, ref_rows=0)


@pytest.mark.parametrize("fmt", ("q4k", "q5k", "q6k"))
def test_gemv_by_name_with_reference_launch_config(gpu, coracle, fmt):
    """CudaModule + launch_kernel(name, grid=N x block=32): the library substitutes its own geometry."""
    ctx, _ = gpu
    mod = t.CudaModule.from_builtin(ctx)
    _check(gpu, coracle, fmt, 515, 2048, seed=5, by_name=mod, ref_rows=0)
    n, k = 300, 1024
    buf, x = kq.gen_matrix(fmt, 9, n, k), kq.gen_x(10, k)
    a = gpu_gemv(gpu, fmt, buf, x, k, n, by_name=mod)
    b = gpu_gemv(gpu, fmt, buf, x, k, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert mod.has_function(f"{fmt}_gemv_warp_reduce")


@pytest.mark.parametrize("fmt", ("q4k", "q5k", "q6k"))
def test_gemv_misaligned_operands(gpu, coracle, fmt):
    """weights at an odd byte offset / x at a 4-byte (not 16-byte) offset take the byte-load kernel."""
    n, k = 129, 1024
    buf, x = kq.gen_matrix(fmt, 21, n, k), kq.gen_x(22, k)
    y64 = kq.gemv_fp64(kq.dequant_matrix(fmt, buf, n, k), x)
    for w_off, x_off in ((1, 0), (0, 1), (6, 3)):
        y = gpu_gemv(gpu, fmt, buf, x, k, n, w_offset=w_off, x_offset=x_off)
        assert kq.rel_l2(y, y64) <= TOL, (w_off, x_off)


@pytest.mark.parametrize("fmt", ("q4k", "q5k", "q6k"))
def test_gemv_deterministic(gpu, fmt):
    n, k = 4096, 4096
    buf, x = kq.gen_matrix(fmt, 31, n, k), kq.gen_x(32, k)
    a = gpu_gemv(gpu, fmt, buf, x, k, n)
    b = gpu_gemv(gpu, fmt, buf, x, k, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))


@pytest.mark.parametrize("fmt", ("q4k", "q5k", "q6k"))
def test_gemv_closed_forms(gpu, fmt):
    """x = 0 gives y = 0; x = e_j picks column j of the dequantised matrix exactly."""
    n, k = 64, 512
    buf = kq.gen_matrix(fmt, 41, n, k)
    w = kq.dequant_matrix(fmt, buf, n, k)
    assert np.array_equal(gpu_gemv(gpu, fmt, buf, np.zeros(k, np.float32), k, n), np.zeros(n, np.float32))
    for j in (0, 31, 32, 255, 256, 300, 511):
        e = np.zeros(k, np.float32)
        e[j] = 1.0
        y = gpu_gemv(gpu, fmt, buf, e, k, n)
        # factorised evaluation: (d*s)*q - dmin*m for Q4/Q5 (one rounding, same as the decode),
        # (d*sc)*(q-32) for Q6 (exact)
        assert np.array_equal(y, w[:, j]), j


def test_gemv_edge_sizes(gpu):
    ctx, stream = gpu
    x = t.GpuBuffer.from_host(ctx, np.ones(256, np.float32))
    w = t.GpuBuffer.from_host(ctx, np.zeros(144, np.uint8))
    y = t.GpuBuffer.from_host(ctx, np.full(4, 7.0, np.float32))
    t.Q4KGemvKernel(256, 0).launch(stream, y, w, x)            # n = 0: nothing written
    stream.synchronize()
    assert np.all(y.copy_to_host() == 7.0)
    t.Q4KGemvKernel(0, 4).launch(stream, y, w, x)              # k = 0: empty sums
    stream.synchronize()
    assert np.all(y.copy_to_host() == 0.0)
    with pytest.raises(t.GpuError) as e:                       # k not a multiple of 256
        t.Q4KGemvKernel(100, 4).launch(stream, y, w, x)
    assert e.value.kind == "KernelLaunch"


def test_gemv_linearity_full_size(gpu):
    """size-independent property at a benchmark shape: W(ax1 + bx2) = a W x1 + b W x2 (to rounding)."""
    n, k = 11008, 4096
    buf = kq.gen_matrix("q4k", 51, n, k)
    x1, x2 = kq.gen_x(52, k), kq.gen_x(53, k)
    y1 = gpu_gemv(gpu, "q4k", buf, x1, k, n).astype(np.float64)
    y2 = gpu_gemv(gpu, "q4k", buf, x2, k, n).astype(np.float64)
    y12 = gpu_gemv(gpu, "q4k", buf, (2.0 * x1 - 0.5 * x2).astype(np.float32), k, n)
    assert kq.rel_l2(y12, 2.0 * y1 - 0.5 * y2) <= 5e-6


@pytest.mark.parametrize("n,k", [(4096, 4096), (32000, 4096), (515, 2048), (129, 1024), (64, 256), (1001, 4096), (2, 4096),
                                 (4097, 3840)])
def test_q6k_streamed_through_lds_gives_the_bits_of_the_register_form(gpu, n, k):
    """Q6_K rows streamed through LDS (opt-in: "gemv_stream_q6k") lie there with their 210-byte blocks re-spaced to 224;
    the arithmetic is the register form's, so every bit must be.  Weights at several alignments (a block may start at any
    even address), ragged row counts (the last batch of a matrix starts early), short rows (fewer pieces than a slot)."""
    tune = lambda key, v: _ffi.lib().trn_set_tuning(key.encode(), int(v))
    buf, x = kq.gen_matrix("q6k", 100 + n, n, k), kq.gen_x(7, k)
    for w_off in (0, 2, 6):
        a = gpu_gemv(gpu, "q6k", buf, x, k, n, w_offset=w_off)
        assert tune("gemv_stream_q6k", 1) == 0 and tune("gemv_stream_min_rows", 1) == 0
        try:
            b = gpu_gemv(gpu, "q6k", buf, x, k, n, w_offset=w_off)
        finally:
            tune("gemv_stream_q6k", 0)
            tune("gemv_stream_min_rows", 0)
        assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), (n, k, w_off)
