"""GPU test of trn_q4k_gemm_noalloc, the Q4_K GEMM entry point that allocates nothing: its results must equal
trn_q4k_gemm's bit for bit (same kernels, the scratch buffer is the library's static device array instead of a
per-stream allocation) and stay within 1e-5 relative L2 of fp64, on two calls in a row, the second with a smaller
input; a product that needs more scratch than the array holds is refused with TRN_ERROR_SCRATCH_TOO_SMALL."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import _ffi

pytestmark = pytest.mark.gpu
TOL = 1e-5


def _both(gpu, m, n, k, seed):
    ctx, stream = gpu
    L = _ffi.lib()
    buf, a = kq.gen_matrix("q4k", seed, n, k), kq.gen_x(seed + 1, m, k)
    dw, da = t.GpuBuffer.from_host(ctx, buf), t.GpuBuffer.from_host(ctx, a)
    out = []
    for fn in (L.trn_q4k_gemm_noalloc, L.trn_q4k_gemm):
        dc = t.GpuBuffer.from_host(ctx, np.full(m * n, np.nan, np.float32))
        rc = fn(stream.raw(), da.as_ptr(), dw.as_ptr(), dc.as_ptr(), m, n, k)
        assert rc == 0, (fn.__name__, rc)
        stream.synchronize()
        out.append(dc.copy_to_host().reshape(m, n))
    ref = kq.gemm_fp64(a, kq.dequant_matrix("q4k", buf, n, k))
    return out[0], out[1], ref


def test_noalloc_gemm_equals_the_allocating_entry_point_twice_in_a_row(gpu):
    # K cut in several parts (the scratch buffer is really used), then a smaller product on the same buffer
    # (all on the matrix cores: more than 8 tokens; the third is the cut with the most partial sums that the library
    # chooses among these shapes: 8 parts of K, 29 groups of 12 strips, 2 token tiles = 11.4 MB)
    for m, n, k, seed in ((16, 1024, 4096, 900), (12, 300, 1024, 910), (32, 11008, 4096, 930)):
        print(f"noalloc case m={m} n={n} k={k}", flush=True)
        got, want, ref = _both(gpu, m, n, k, seed)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), (m, n, k)
        assert kq.rel_l2(got, ref) <= TOL
    # m = 1 and unaligned operands take the kernels without scratch: still the same results
    got, want, ref = _both(gpu, 1, 257, 512, 920)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)) and kq.rel_l2(got, ref) <= TOL
    # so do three tokens against 14336 rows (the integer matrix cores: no scratch either)
    got, want, ref = _both(gpu, 3, 14336, 4096, 940)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32)) and kq.rel_l2(got, ref) <= TOL


def test_noalloc_gemm_refuses_what_does_not_fit(gpu):
    ctx, stream = gpu
    L = _ffi.lib()
    m, n, k = 16, 2048, 65536                     # with K forced into 256 parts: 8 x 256 x 16 KB of partial results, twice the array
    dw = t.GpuBuffer(ctx, n * (k // 256) * 144, np.uint8)
    da = t.GpuBuffer(ctx, m * k, np.float32)
    dc = t.GpuBuffer(ctx, m * n, np.float32)
    assert L.trn_set_tuning(b"gemm_k_parts", 1024) == 0
    try:
        rc = L.trn_q4k_gemm_noalloc(stream.raw(), da.as_ptr(), dw.as_ptr(), dc.as_ptr(), m, n, k)
    finally:
        L.trn_set_tuning(b"gemm_k_parts", 0)
    stream.synchronize()
    assert rc == 9002 and L.trn_error_name(rc) == b"TRN_ERROR_SCRATCH_TOO_SMALL"
    assert L.trn_q4k_gemm_noalloc(stream.raw(), da.as_ptr(), dw.as_ptr(), dc.as_ptr(), m, n, 100) == 1
