"""The legacy "simplified" Q4_K format of q4k_gemm_fused (18-byte blocks of 32 values, quantize.rs:41, 151-336):
oracle pins on the CPU, parity of the GPU kernel through the C ABI."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import kernels as K


def _block(scale_f16_bits: int, nibble_bytes) -> np.ndarray:
    b = np.zeros(18, np.uint8)
    b[0], b[1] = scale_f16_bits & 255, scale_f16_bits >> 8
    b[2:] = nibble_bytes
    return b


# ---- oracle pins (no GPU) ---------------------------------------------------------------------

def test_constants_follow_the_reference():
    # quantize.rs:34, 41: 32 values in 18 bytes = 2 (f16 scale) + 16 (nibbles)
    assert kq.Q4K_SIMPLE_BLOCK == 32 and kq.Q4K_SIMPLE_BYTES == 18 == 2 + 32 // 2
    assert t.QuantizeKernel(4, 8, 64).num_blocks_per_row() == 2
    assert t.QuantizeKernel(4, 8, 64).weight_bytes() == 8 * 2 * 18


def test_scale_one_gives_the_quants_in_sequential_nibble_order():
    # scale = 1.0 (f16 0x3C00): w_i = q_i; value i is byte i/2, low nibble for even i (quantize.rs:245-262)
    nib = np.arange(16, dtype=np.uint8) | (((15 - np.arange(16)) << 4).astype(np.uint8))
    w = kq.dequant_q4k_simplified(_block(0x3C00, nib))[0]
    assert np.array_equal(w[0::2], np.arange(16, dtype=np.float32))
    assert np.array_equal(w[1::2], (15 - np.arange(16)).astype(np.float32))


def test_one_hot_bit_map():
    # every one of the 128 quant bits moves exactly one value by scale * 2^(bit within its nibble)
    scale = np.float32(np.float16(0.5))
    for bit in range(128):
        nib = np.zeros(16, np.uint8)
        nib[bit // 8] = 1 << (bit % 8)
        w = kq.dequant_q4k_simplified(_block(0x3800, nib))[0]      # 0x3800 = 0.5
        i = 2 * (bit // 8) + (bit % 8) // 4
        expect = np.zeros(32, np.float32)
        expect[i] = scale * (1 << (bit % 4))
        assert np.array_equal(w, expect), bit


def test_no_min_term_and_exactness():
    rng = np.random.default_rng(5)
    buf = kq.gen_q4k_simplified(rng, 300)
    w = kq.dequant_q4k_simplified(buf)
    b = buf.reshape(-1, 18)
    assert np.all(w[(np.repeat(b[:, 2:], 2, axis=1) >> np.tile([0, 4], 16) & 15) == 0] == 0.0)   # q = 0 -> w = 0
    # f16 scale (11 bits) x 4-bit quant is exact in f32: fp64 evaluation rounds to the same bits
    s64 = b[:, 0:2].copy().view(np.float16).astype(np.float64)
    q = np.empty((b.shape[0], 32)); q[:, 0::2] = b[:, 2:] & 15; q[:, 1::2] = b[:, 2:] >> 4
    assert np.array_equal((s64 * q).astype(np.float32), w)


def test_numpy_and_c_restatements_agree(coracle):
    buf = kq.gen_q4k_simplified(np.random.default_rng(6), 1000)
    assert np.array_equal(kq.dequant_q4k_simplified(buf).view(np.uint32), coracle.dequant_simplified(buf).view(np.uint32))
    m, n, k = 3, 7, 96
    wbuf = kq.gen_q4k_simplified(np.random.default_rng(7), n * k // 32)
    a = kq.gen_x(8, m, k)
    c_np = kq.gemm_fp64(a, kq.dequant_matrix_simplified(wbuf, n, k))
    assert np.allclose(coracle.gemm_simplified_fp64(wbuf, a, m, n, k), c_np, rtol=1e-12, atol=1e-12)


def test_brute_force_tiny_gemm():
    # one block per row, scale 1: C[r][col] = sum_i q[col][i] * a[r][i], by hand
    n, k, m = 2, 32, 2
    nib = np.stack([np.full(16, 0x21, np.uint8), np.full(16, 0xF0, np.uint8)])
    buf = np.concatenate([_block(0x3C00, nib[0]), _block(0x3C00, nib[1])])
    a = np.stack([np.ones(32, np.float32), np.arange(32, dtype=np.float32)])
    c = kq.gemm_fp64(a, kq.dequant_matrix_simplified(buf, n, k))
    q0 = np.tile([1.0, 2.0], 16); q1 = np.tile([0.0, 15.0], 16)
    assert np.array_equal(c, np.array([[q0.sum(), q1.sum()], [q0 @ np.arange(32), q1 @ np.arange(32)]]))


# ---- GPU parity --------------------------------------------------------------------------------

TOL = 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("n_blocks", (1, 33, 4096))
def test_gpu_dequant_bit_exact(gpu, n_blocks):
    ctx, stream = gpu
    buf = kq.gen_q4k_simplified(np.random.default_rng(20 + n_blocks), n_blocks)
    dw = t.GpuBuffer.from_host(ctx, buf)
    out = t.GpuBuffer.from_host(ctx, np.full(n_blocks * 32, np.nan, np.float32))
    K.dequant_simplified_f32(stream, out, dw, n_blocks)
    stream.synchronize()
    assert np.array_equal(out.copy_to_host().view(np.uint32), kq.dequant_q4k_simplified(buf).reshape(-1).view(np.uint32))


@pytest.mark.gpu
@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (4, 1000, 2048), (16, 333, 32), (64, 64, 4128), (3, 5, 64)])
@pytest.mark.parametrize("by_name", (False, True))
def test_gpu_gemm_fused_against_fp64(gpu, m, n, k, by_name):
    ctx, stream = gpu
    buf = kq.gen_q4k_simplified(np.random.default_rng(30 + m), n * k // 32)
    a = kq.gen_x(31 + m, m, k)
    dw, da = t.GpuBuffer.from_host(ctx, buf), t.GpuBuffer.from_host(ctx, a.reshape(-1))
    dc = t.GpuBuffer.from_host(ctx, np.full(m * n, np.nan, np.float32))
    kern = t.QuantizeKernel(m, n, k)
    assert kern.name() == "q4k_gemm_fused"
    if by_name:
        kern.launch_by_name(stream, t.CudaModule.from_builtin(ctx), da, dw, dc)    # the caller's geometry is replaced
    else:
        kern.launch(stream, da, dw, dc)
    stream.synchronize()
    c = dc.copy_to_host().reshape(m, n)
    assert kq.rel_l2(c, kq.gemm_fp64(a, kq.dequant_matrix_simplified(buf, n, k))) <= TOL


@pytest.mark.gpu
def test_gpu_gemm_fused_edge_cases(gpu):
    ctx, stream = gpu
    a = t.GpuBuffer.from_host(ctx, np.ones(64, np.float32))
    w = t.GpuBuffer.from_host(ctx, np.zeros(36, np.uint8))
    c = t.GpuBuffer.from_host(ctx, np.full(4, 3.0, np.float32))
    t.QuantizeKernel(0, 1, 64).launch(stream, a, w, c)
    t.QuantizeKernel(1, 0, 64).launch(stream, a, w, c)
    stream.synchronize()
    assert np.all(c.copy_to_host() == 3.0)
    with pytest.raises(t.GpuError):
        t.QuantizeKernel(1, 1, 48).launch(stream, a, w, c)       # k % 32 != 0
