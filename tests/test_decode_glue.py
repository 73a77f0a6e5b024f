"""The element-wise decoder-layer kernels (elementwise.rs: residual_add, fused_residual_rmsnorm, fused_swiglu;
layernorm.rs: rmsnorm): oracle pins on the CPU, parity of the GPU kernels through the C ABI.

Tolerances.  residual_add is bit-exact.  The other three contain one approximate instruction each in the reference
(ex2.approx, rsqrt.approx: 2^-22 relative by the PTX manual) next to individually rounded f32 operations, so the
reference's own result lies within about 2^-22 + 3 * 2^-24 of the oracle's exact evaluation; the GPU kernels are
held to REL = 6e-7 of it (plus ABS for results that underflow)."""
import ctypes as C

import numpy as np
import pytest

import trueno_amd as t
from oracle import glue

REL, ABS = 6e-7, 1e-37


def _close(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return np.all(np.abs(got - want) <= REL * np.abs(want) + ABS)


# ---- oracle pins (no GPU) ---------------------------------------------------------------------

def test_names_and_defaults_follow_the_reference():
    assert t.ResidualAddKernel(8).name() == "residual_add"                      # elementwise.rs:47-49
    assert t.FusedSwigluKernel(8).name() == "fused_swiglu"                      # :535-537
    assert t.RmsNormKernel(8).name() == "rmsnorm"                               # layernorm.rs:414-416
    assert t.FusedResidualRmsNormKernel(8).name() == "fused_residual_rmsnorm"   # elementwise.rs:135-137
    assert t.RmsNormKernel(8).epsilon == 1e-5 and t.FusedResidualRmsNormKernel(8).epsilon == 1e-5
    assert t.RmsNormKernel(8).with_epsilon(1e-6).epsilon == 1e-6
    assert t.ResidualAddKernel(1000).launch_config().grid == (4, 1, 1)           # ceil(n / 256) blocks of 256
    assert t.RmsNormKernel(4096).launch_config().block == (32, 1, 1)             # one warp


def test_swiglu_closed_forms():
    up = np.float32(3.0)
    assert glue.fused_swiglu([0.0], [up])[0] == 0.0                              # silu(0) = 0
    assert glue.fused_swiglu([40.0], [up])[0] == np.float32(120.0)               # sigmoid(40) rounds to 1
    assert glue.fused_swiglu([-200.0], [up])[0] == 0.0                           # 2^(+288) overflows: 1/inf = 0
    g = np.linspace(-20, 20, 4001).astype(np.float32)
    s_pos, s_neg = glue.fused_swiglu(g, np.ones_like(g)), glue.fused_swiglu(-g, np.ones_like(g))
    assert np.max(np.abs((s_pos - s_neg) - g)) <= 4e-6                           # silu(g) - silu(-g) = g
    # against the textbook formula: the literal 1.442695f is log2(e) to 2e-8 relative, which at |g| <= 20 moves
    # the exponent by at most 20 * 1.4427 * 2e-8 * ln 2 = 4e-7 relative
    want = glue.fused_swiglu_fp64(g, np.full_like(g, 1.5))
    got = glue.fused_swiglu(g, np.full_like(g, 1.5))
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-30)) <= 1e-6


def test_rmsnorm_closed_forms():
    n = 96
    gamma = np.linspace(0.5, 2.0, n).astype(np.float32)
    # a constant row c: mean square c^2, output c / sqrt(c^2 + eps) * gamma
    c, eps = np.float32(3.0), 1e-5
    want = np.float64(c) / np.sqrt(np.float64(c) ** 2 + np.float64(np.float32(eps))) * gamma.astype(np.float64)
    got = glue.rmsnorm(np.full(n, c, np.float32), gamma, eps)
    assert np.max(np.abs(got - want) / want) <= 3e-7
    # a one-hot row: mean square v^2 / n
    x = np.zeros(n, np.float32)
    x[17] = 4.0
    got = glue.rmsnorm(x, gamma, 0.0)
    assert np.all(got[np.arange(n) != 17] == 0.0)
    assert abs(got[17] - np.sqrt(n) * gamma[17]) <= 3e-7 * np.sqrt(n) * gamma[17]
    # gamma = 1: the output's mean square is ms / (ms + eps); scaling the input by 2^k changes nothing but eps's weight
    rng = np.random.default_rng(3)
    x = rng.standard_normal(1000).astype(np.float32)
    y = glue.rmsnorm(x, np.ones(1000, np.float32), 0.0).astype(np.float64)
    assert abs(np.mean(y * y) - 1.0) <= 1e-6
    assert np.array_equal(glue.rmsnorm(x * np.float32(1024.0), np.ones(1000, np.float32), 0.0),
                          glue.rmsnorm(x, np.ones(1000, np.float32), 0.0))
    # the lane order against fp64
    g = rng.standard_normal(1000).astype(np.float32)
    want = glue.rmsnorm_fp64(x, g)
    assert np.max(np.abs(glue.rmsnorm(x, g) - want) / np.maximum(np.abs(want), 1e-30)) <= 4e-7
    # with a residual the sum is an f32 add first
    r = rng.standard_normal(1000).astype(np.float32)
    assert np.array_equal(glue.rmsnorm(x, g, residual=r), glue.rmsnorm((x + r).astype(np.float32), g))


def test_sum_of_squares_lane_order():
    # 64 ones: lanes 0..31 hold 2 each, the tree adds them to 64; a value only lane 5 sees
    assert glue.sum_squares_ref_order(np.ones(64, np.float32)) == 64.0
    x = np.zeros(70, np.float32)
    x[5], x[37], x[69] = 1.0, 2.0, 3.0
    assert glue.sum_squares_ref_order(x) == 14.0


# ---- GPU parity (C ABI) ---------------------------------------------------------------------

def _dev(gpu, a):
    return t.GpuBuffer.from_host(gpu[0], np.ascontiguousarray(a, np.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("n", (1, 255, 256, 257, 4096, 11008, 100003))
def test_gpu_residual_add_is_exact(gpu, n):
    rng = np.random.default_rng(n)
    a, b = rng.standard_normal(n).astype(np.float32), (rng.standard_normal(n) * 1e3).astype(np.float32)
    da, db, do = _dev(gpu, a), _dev(gpu, b), _dev(gpu, np.zeros(n))
    t.ResidualAddKernel(n).launch(gpu[1], da, db, do)
    gpu[1].synchronize()
    assert np.array_equal(do.copy_to_host().view(np.uint32), glue.residual_add(a, b).view(np.uint32))
    t.ResidualAddKernel(n).launch(gpu[1], da, db, da)                  # output aliases input1 (x = x + f(x))
    gpu[1].synchronize()
    assert np.array_equal(da.copy_to_host().view(np.uint32), glue.residual_add(a, b).view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("n", (1, 257, 11008, 28672))
def test_gpu_fused_swiglu(gpu, n):
    rng = np.random.default_rng(100 + n)
    gate = (rng.standard_normal(n) * 4).astype(np.float32)
    gate[: min(n, 6)] = np.array([0.0, -0.0, 40.0, -40.0, 100.0, -200.0], np.float32)[: min(n, 6)]
    up = rng.standard_normal(n).astype(np.float32)
    dg, du, do = _dev(gpu, gate), _dev(gpu, up), _dev(gpu, np.zeros(n))
    t.FusedSwigluKernel(n).launch(gpu[1], dg, du, do)
    gpu[1].synchronize()
    assert _close(do.copy_to_host(), glue.fused_swiglu(gate, up))


@pytest.mark.gpu
@pytest.mark.parametrize("hidden", (1, 31, 64, 1000, 4096, 11008))
@pytest.mark.parametrize("residual", (False, True))
def test_gpu_rmsnorm(gpu, hidden, residual):
    rng = np.random.default_rng(200 + hidden)
    x = (rng.standard_normal(hidden) * 3).astype(np.float32)
    r = rng.standard_normal(hidden).astype(np.float32) if residual else None
    gamma = rng.uniform(0.5, 1.5, hidden).astype(np.float32)
    dx, dg, do = _dev(gpu, x), _dev(gpu, gamma), _dev(gpu, np.zeros(hidden))
    if residual:
        dr = _dev(gpu, r)
        t.FusedResidualRmsNormKernel(hidden).launch(gpu[1], dr, dx, do, dg)
    else:
        t.RmsNormKernel(hidden).with_epsilon(1e-6).launch(gpu[1], dx, do, dg)
    gpu[1].synchronize()
    want = glue.rmsnorm(x, gamma, 1e-5 if residual else 1e-6, residual=r)
    got = do.copy_to_host()
    # the sum of squares is added in another order than the reference's 32 lanes: a few 2^-24 of the total
    assert np.all(np.abs(got.astype(np.float64) - want) <= (REL + 3e-7) * np.abs(want) + ABS)
    assert np.max(np.abs(got - glue.rmsnorm_fp64(x, gamma, 1e-5 if residual else 1e-6, residual=r))
                  / np.maximum(np.abs(want), 1e-30)) <= 1e-6
    # in place: output aliases the input (the residual), as the reference allows
    if residual:
        t.FusedResidualRmsNormKernel(hidden).launch(gpu[1], dr, dx, dr, dg)
        gpu[1].synchronize()
        assert np.array_equal(dr.copy_to_host().view(np.uint32), got.view(np.uint32))
    else:
        t.RmsNormKernel(hidden).with_epsilon(1e-6).launch(gpu[1], dx, dx, dg)
        gpu[1].synchronize()
        assert np.array_equal(dx.copy_to_host().view(np.uint32), got.view(np.uint32))


@pytest.mark.gpu
def test_gpu_glue_by_name_with_the_references_geometry(gpu):
    ctx, stream = gpu
    module = t.CudaModule.from_builtin(ctx)
    n = 5000
    rng = np.random.default_rng(7)
    a, b, gamma = (rng.standard_normal(n).astype(np.float32) for _ in range(3))
    da, db, dg, do = _dev(gpu, a), _dev(gpu, b), _dev(gpu, gamma), _dev(gpu, np.zeros(n))
    t.ResidualAddKernel(n).launch_by_name(stream, module, da, db, do)
    stream.synchronize()
    assert np.array_equal(do.copy_to_host(), glue.residual_add(a, b))
    t.FusedSwigluKernel(n).launch_by_name(stream, module, da, db, do)
    stream.synchronize()
    assert _close(do.copy_to_host(), glue.fused_swiglu(a, b))
    t.RmsNormKernel(n).launch_by_name(stream, module, da, do, dg)
    stream.synchronize()
    assert np.all(np.abs(do.copy_to_host() - glue.rmsnorm(a, gamma)) <= 1e-6 * np.abs(glue.rmsnorm(a, gamma)) + ABS)
    t.FusedResidualRmsNormKernel(n).launch_by_name(stream, module, da, db, do, dg)
    stream.synchronize()
    want = glue.rmsnorm(b, gamma, residual=a)
    assert np.all(np.abs(do.copy_to_host() - want) <= 1e-6 * np.abs(want) + ABS)


@pytest.mark.gpu
def test_gpu_glue_edge_cases(gpu):
    ctx, stream = gpu
    L = t._ffi.lib()
    d = _dev(gpu, np.full(8, 2.0))
    assert L.trn_residual_add(stream.raw(), d.as_ptr(), d.as_ptr(), d.as_ptr(), 0) == 0        # n = 0: nothing happens
    assert L.trn_rmsnorm(stream.raw(), d.as_ptr(), d.as_ptr(), d.as_ptr(), 0, C.c_float(1e-5)) == 0
    stream.synchronize()
    assert np.all(d.copy_to_host() == 2.0)
    assert L.trn_residual_add(stream.raw(), 0, d.as_ptr(), d.as_ptr(), 8) != 0                 # null pointer
    assert L.trn_fused_residual_rmsnorm(stream.raw(), 0, d.as_ptr(), d.as_ptr(), d.as_ptr(), 8, C.c_float(1e-5)) != 0
