"""GPU parity, batched GEMM C = A . dequant(W)^T: within 1e-5 relative L2 of fp64 for M in {1, 4, 16, 64},
row-major C, m = 1 equal to the GEMV; typed launcher and launch-by-name."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from tests.kq_helpers import REF_SLACK, gpu_gemm, gpu_gemv, record_ratio

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


@pytest.mark.parametrize("m", (1, 5))
@pytest.mark.parametrize("fmt,n,k", [("q4k", 300, 1024), ("q5k", 300, 1024), ("q6k", 300, 2048), ("q4k", 64, 14336)])
def test_gemm_with_the_decode_as_written(gpu, fmt, n, k, m):
    """q*k_gemm_ggml with the GEMM family's own decode (policy 1; quantize.rs:445-514, :727-807, :1009-1064): against
    fp64 on the oracle's as-written weights, and really different from the canonical decode's product."""
    buf, a = kq.gen_matrix(fmt, 400 + m, n, k), kq.gen_x(500 + m, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k, as_written=True)
    want = kq.gemm_fp64(a, kq.dequant_matrix(fmt, buf, n, k, policy=1))
    assert c.shape == (m, n) and np.all(np.isfinite(c))
    assert kq.rel_l2(c, want) <= TOL
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) > 1e-2


@pytest.mark.parametrize("m", (1, 4, 16, 64))
def test_gemm_config_shape_w_14336x4096(gpu, m):
    n, k = 14336, 4096
    buf, a = kq.gen_matrix("q4k", 1234, n, k), kq.gen_x(4321, m, k)
    c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
    assert kq.rel_l2(c, _c64("q4k", buf, a, n, k)) <= TOL


@pytest.mark.parametrize("m", (1, 4, 16, 64))
def test_gemm_config_shape_w_4096x14336(gpu, m):
    n, k = 4096, 14336
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


def _tune(key, value):
    from trueno_amd import _ffi
    assert _ffi.lib().trn_set_tuning(key.encode(), int(value)) == 0


MFMA_FORMATS = ("q4k", "q5k", "q6k")      # the formats whose GEMM runs on the matrix cores for m >= 2


@pytest.mark.parametrize("m", (4, 16, 64))
@pytest.mark.parametrize("fmt", ("q5k", "q6k"))
def test_gemm_4096x4096(gpu, fmt, m):
    n = k = 4096
    buf, a = kq.gen_matrix(fmt, 1239, n, k), kq.gen_x(4321, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL


@pytest.mark.parametrize("m", (2, 9, 13, 33))
@pytest.mark.parametrize("n,k", [(100, 512), (1000, 2304)])
@pytest.mark.parametrize("fmt", MFMA_FORMATS)
def test_gemm_matrix_core_form_ragged(gpu, fmt, n, k, m):
    """Token counts that do not fill a tile of 16, row counts that do not fill a strip of 32 or a group of 8 strips."""
    buf, a = kq.gen_matrix(fmt, 50 + m, n, k), kq.gen_x(60 + m, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL


@pytest.mark.parametrize("m", (17, 33, 40, 64))
@pytest.mark.parametrize("fmt", ("q4k", "q5k"))
def test_gemm_two_token_tiles_per_workgroup(gpu, fmt, m):
    """The kernels that take two tiles of 16 tokens per workgroup, forced on a small product: odd numbers of tiles
    (the second tile of the last pair does not exist), K in one part and in several, the same bits on every run;
    and one tile per workgroup gives the same bits for the same cut of K (a tile's sums do not depend on its
    company)."""
    n, k = 300, 1536
    buf, a = kq.gen_matrix(fmt, 70 + m, n, k), kq.gen_x(80 + m, m, k)
    c64 = _c64(fmt, buf, a, n, k)
    try:
        for parts in (1, 3):
            _tune("gemm_k_parts", parts)
            _tune("gemm_tiles", 2)
            two = gpu_gemm(gpu, fmt, buf, a, m, n, k)
            assert kq.rel_l2(two, c64) <= TOL
            again = gpu_gemm(gpu, fmt, buf, a, m, n, k)
            assert np.array_equal(again.view(np.uint32), two.view(np.uint32)), parts
            _tune("gemm_tiles", 1)
            one = gpu_gemm(gpu, fmt, buf, a, m, n, k)
            assert np.array_equal(one.view(np.uint32), two.view(np.uint32)), parts
    finally:
        _tune("gemm_k_parts", 0)
        _tune("gemm_tiles", 0)


@pytest.mark.parametrize("fmt", ("q4k", "q5k"))
def test_gemm_many_tokens(gpu, fmt):
    """512 tokens against 4096 x 2048: enough workgroups that the library itself takes two tiles per workgroup."""
    n, k, m = 4096, 2048, 512
    buf, a = kq.gen_matrix(fmt, 77, n, k), kq.gen_x(78, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL


@pytest.mark.parametrize("m", (5, 20))
@pytest.mark.parametrize("fmt", MFMA_FORMATS)
def test_gemm_few_rows_long_k(gpu, fmt, m):
    """96 rows against K = 8192: one group of strips, so the library cuts K into as many parts as there are
    super-blocks (32) and the last workgroup adds them in two rounds of sixteen."""
    n, k = 96, 8192
    buf, a = kq.gen_matrix(fmt, 300 + m, n, k), kq.gen_x(310 + m, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL
    again = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert np.array_equal(again.view(np.uint32), c.view(np.uint32))


@pytest.mark.parametrize("m", (5, 24, 40))
def test_gemm_twelve_strips_per_workgroup(gpu, m):
    """The Q4_K kernel that takes twelve strips of 32 rows per workgroup (its last four waves convert no tokens), forced
    on a small product whose rows fill neither the last strip nor the last workgroup: within tolerance, and the same
    bits as eight strips per workgroup for the same cut of K (a strip's sums do not depend on its company)."""
    n, k = 777, 2048
    buf, a = kq.gen_matrix("q4k", 400 + m, n, k), kq.gen_x(410 + m, m, k)
    c64 = _c64("q4k", buf, a, n, k)
    try:
        for parts in (1, 3):
            _tune("gemm_k_parts", parts)
            _tune("gemm_waves", 12)
            twelve = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
            assert kq.rel_l2(twelve, c64) <= TOL
            _tune("gemm_waves", 8)
            _tune("gemm_tiles", 1)
            eight = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
            assert np.array_equal(eight.view(np.uint32), twelve.view(np.uint32)), parts
            _tune("gemm_tiles", 0)
    finally:
        _tune("gemm_k_parts", 0)
        _tune("gemm_waves", 0)
        _tune("gemm_tiles", 0)


@pytest.mark.parametrize("m", (4, 32))
@pytest.mark.parametrize("fmt", MFMA_FORMATS)
def test_gemm_ffn_shape_w_11008x4096(gpu, fmt, m):
    """The 7B gate/up shape: 43 groups of 8 strips do not divide the CUs well, so the library takes fewer parts of K than
    would fill them (and, for Q4_K with 32 tokens, twelve strips per workgroup)."""
    n, k = 11008, 4096
    buf, a = kq.gen_matrix(fmt, 500 + m, n, k), kq.gen_x(510 + m, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL


def _random_shapes():
    rng = np.random.default_rng(20251125)
    for i in range(15):
        fmt = MFMA_FORMATS[i % 3]
        k = 256 * int(rng.integers(1, 33))
        n = int(rng.integers(1, 5000)) if i % 3 else 32 * int(rng.integers(1, 150))
        m = int(rng.choice([2, 3, 5, 9, 16, 17, 31, 33, 48, 64, 65, 100, 130, 257]))
        yield fmt, m, n, k, i


@pytest.mark.parametrize("fmt,m,n,k,i", list(_random_shapes()))
def test_gemm_random_shapes(gpu, fmt, m, n, k, i):
    """Shapes drawn at random (fixed seed): whatever cut of the product the library's estimate picks for them - strips per
    workgroup, token tiles per workgroup, parts of K of unequal length - the result is within tolerance."""
    buf, a = kq.gen_matrix(fmt, 1000 + i, n, k), kq.gen_x(2000 + i, m, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    assert np.all(np.isfinite(c))
    assert kq.rel_l2(c, _c64(fmt, buf, a, n, k)) <= TOL


@pytest.mark.parametrize("fmt", MFMA_FORMATS)
def test_gemm_parts_of_k(gpu, fmt):
    """However K is cut into parts the result stays within tolerance, and the same cut gives the same bits on
    every run: the parts are added in part order by whichever workgroup arrives last."""
    n, k, m = 777, 2048, 24
    buf, a = kq.gen_matrix(fmt, 91, n, k), kq.gen_x(92, m, k)
    c64 = _c64(fmt, buf, a, n, k)
    try:
        for waves in (4, 8):
            _tune("gemm_waves", waves)
            for parts in (1, 2, 3, 8):
                _tune("gemm_k_parts", parts)
                first = gpu_gemm(gpu, fmt, buf, a, m, n, k)
                assert kq.rel_l2(first, c64) <= TOL
                for _ in range(3):
                    again = gpu_gemm(gpu, fmt, buf, a, m, n, k)
                    assert np.array_equal(again.view(np.uint32), first.view(np.uint32)), (waves, parts)
    finally:
        _tune("gemm_k_parts", 0)
        _tune("gemm_waves", 0)
    try:
        _tune("gemm_mfma_off", 1)
        valu = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    finally:
        _tune("gemm_mfma_off", 0)
    assert kq.rel_l2(valu, c64) <= TOL


# The matrix-core form against the reference's own f32 result, per format and cut: (shape, tokens).  4096 columns in one
# part, 14336 columns in parts of K; 16 tokens (one tile) and 64 (two tiles per workgroup for Q4_K / Q5_K).
@pytest.mark.parametrize("n,k,m", [(2048, 4096, 16), (1024, 14336, 16), (1024, 4096, 64)])
@pytest.mark.parametrize("fmt", MFMA_FORMATS)
def test_gemm_no_worse_than_reference_order_f32(gpu, coracle, fmt, n, k, m):
    """Per product, the error against fp64 is no larger than that of an f32 evaluation in the reference's summation
    order (quantize.rs:1412-1518), up to the sampling margin."""
    buf, a = kq.gen_matrix(fmt, 93, n, k), kq.gen_x(94, m, k)
    w = kq.dequant_matrix(fmt, buf, n, k)
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    c64 = kq.gemm_fp64(a, w)
    ref = np.stack([coracle.gemv_ref_order_f32(fmt, buf, a[i], k, n) for i in range(m)])
    err_ref, err_ours = kq.rel_l2(ref, c64), kq.rel_l2(c, c64)
    record_ratio("gemm", fmt, m, n, k, n, err_ours, err_ref)
    assert err_ours <= REF_SLACK * err_ref, (fmt, m, n, k, err_ours, err_ref, err_ours / err_ref)


@pytest.mark.parametrize("fmt", MFMA_FORMATS)
def test_gemm_special_values(gpu, fmt):
    """An all-zero token, a huge and a tiny token, and a token with an infinity (its outputs are not finite,
    the other tokens are untouched)."""
    n, k, m = 64, 512, 5
    buf = kq.gen_matrix(fmt, 95, n, k)
    a = kq.gen_x(96, m, k)
    a[1] = 0.0
    a[2] *= 1e30
    a[3] *= 1e-30
    a[4, 17] = np.inf
    c = gpu_gemm(gpu, fmt, buf, a, m, n, k)
    w = kq.dequant_matrix(fmt, buf, n, k)
    c64 = kq.gemm_fp64(a[:4], w)
    assert np.all(c[1] == 0.0)
    for i in (0, 2, 3):
        assert kq.rel_l2(c[i], c64[i]) <= TOL
    assert not np.any(np.isfinite(c[4]))


def test_gemm_on_streams_that_come_and_go(gpu):
    """the scratch buffers a stream's products use (partial sums, arrival counters) go with the stream; a new stream,
    possibly with the old one's handle, starts from clean ones"""
    ctx, _ = gpu
    n, k, m = 1024, 4096, 4                       # K is cut in parts on this shape: partial sums and counters in use
    buf, a = kq.gen_matrix("q4k", 91, n, k), kq.gen_x(92, m, k)
    want = _c64("q4k", buf, a, n, k)
    first = None
    for _ in range(3):
        stream = t.CudaStream(ctx)
        c = gpu_gemm((ctx, stream), "q4k", buf, a, m, n, k)
        assert kq.rel_l2(c, want) <= TOL
        first = c if first is None else first
        assert np.array_equal(c.view(np.uint32), first.view(np.uint32))
        stream.destroy()


# ---- two to four tokens on the integer matrix cores (Q4_K, k <= 4096) --------------------------------------------------
FEW_SHAPES = [(64, 256), (100, 1024), (33, 2304), (1000, 4096), (8300, 4096), (14336, 4096)]


@pytest.mark.parametrize("m", (2, 3, 4))
@pytest.mark.parametrize("n,k", FEW_SHAPES)
def test_gemm_few_tokens_on_the_integer_cores(gpu, n, k, m):
    """One to 260 tiles of 32 rows (one or two per workgroup, the last one ragged), one to sixteen super-blocks per row,
    every token count the kernel takes: within the contract's distance of fp64, and not the result of another path."""
    buf, a = kq.gen_matrix("q4k", 600 + m, n, k), kq.gen_x(700 + m, m, k)
    want = _c64("q4k", buf, a, n, k)
    try:
        _tune("gemm_few", 1)
        c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
        _tune("gemm_few", 2)
        other = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
    finally:
        _tune("gemm_few", 0)
    assert c.shape == (m, n) and np.all(np.isfinite(c))
    assert kq.rel_l2(c, want) <= TOL and kq.rel_l2(other, want) <= TOL
    assert not np.array_equal(c, other)                      # (two orders of summation: the same bits would mean one path ran twice)


@pytest.mark.parametrize("n,k,m", [(20000, 4096, 3), (40000, 4096, 2), (30000, 1024, 4), (70000, 256, 4)])
def test_gemm_few_tokens_several_tiles_per_workgroup(gpu, n, k, m):
    """Three to nine tiles per workgroup: the copies of the tile after next are issued between the products of the
    current one, and a tile's results leave while the next is multiplied (rows of 16, 4 and 1 super-blocks: four, two and
    one of the eight waves have products of their own)."""
    buf, a = kq.gen_matrix("q4k", 810 + m, n, k), kq.gen_x(820 + m, m, k)
    try:
        _tune("gemm_few", 1)
        c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
    finally:
        _tune("gemm_few", 0)
    want = _c64("q4k", buf, a, n, k)
    assert np.all(np.isfinite(c)) and kq.rel_l2(c, want) <= TOL
    for i in range(m):                                       # every token, and the ends of the matrix on their own
        assert kq.rel_l2(c[i], want[i]) <= TOL
        assert kq.rel_l2(c[i, -40:], want[i, -40:]) <= TOL and kq.rel_l2(c[i, :40], want[i, :40]) <= TOL


@pytest.mark.parametrize("m", (2, 4))
def test_gemm_few_tokens_no_worse_than_reference_order_f32(gpu, coracle, m):
    n, k = 2048, 4096
    buf, a = kq.gen_matrix("q4k", 93, n, k), kq.gen_x(94, m, k)
    c64 = kq.gemm_fp64(a, kq.dequant_matrix("q4k", buf, n, k))
    try:
        _tune("gemm_few", 1)
        c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
    finally:
        _tune("gemm_few", 0)
    ref = np.stack([coracle.gemv_ref_order_f32("q4k", buf, a[i], k, n) for i in range(m)])
    err_ref, err_ours = kq.rel_l2(ref, c64), kq.rel_l2(c, c64)
    record_ratio("gemm_few", "q4k", m, n, k, n, err_ours, err_ref)
    assert err_ours <= REF_SLACK * err_ref, (m, err_ours, err_ref, err_ours / err_ref)


def test_gemm_few_tokens_special_values(gpu):
    """Tokens of zeros, of huge and of tiny values; a token whose runs of 256 differ by 2^40 in size and one with a single
    large element among small ones (each run has its own power of two, so the small ones keep their bits); unit vectors
    (the product is then one weight, d * s * q - dmin * m, to a few ulps of its two terms); an infinity spoils its
    token and no other."""
    n, k = 96, 1024
    buf = kq.gen_matrix("q4k", 95, n, k)
    w = kq.dequant_matrix("q4k", buf, n, k)
    a = kq.gen_x(96, 4, k)
    a[1] = 0.0
    a[2] *= 1e30
    a[3, :256] *= 2.0 ** 40
    a[3, 700] = 3.0e4
    try:
        _tune("gemm_few", 1)
        c = gpu_gemm(gpu, "q4k", buf, a, 4, n, k)
        a2 = kq.gen_x(97, 3, k) * 1e-30
        a2[1] = 0.0
        a2[1, 517] = 1.0
        a2[2, 3] = np.inf
        c2 = gpu_gemm(gpu, "q4k", buf, a2.astype(np.float32), 3, n, k)
    finally:
        _tune("gemm_few", 0)
    c64 = kq.gemm_fp64(a, w)
    assert np.all(c[1] == 0.0)
    for i in (0, 2, 3):
        assert kq.rel_l2(c[i], c64[i]) <= TOL
    assert kq.rel_l2(c2[0], kq.gemm_fp64(a2[:1].astype(np.float32), w)[0]) <= TOL
    col = w[:, 517].astype(np.float64)
    assert np.all(np.abs(c2[1] - col) <= 2.0 ** -21 * np.abs(w).max())
    assert not np.any(np.isfinite(c2[2]))


def test_gemm_few_tokens_by_the_rule(gpu):
    """Left to itself the launcher takes the integer-core kernel where it is the fastest way (two tokens against 14336
    rows), and not for one token, for five, or for rows longer than a slab of 4096 columns."""
    for m, n, k, taken in [(2, 14336, 4096, True), (1, 2048, 4096, False), (5, 2048, 4096, False), (2, 256, 8192, False)]:
        buf, a = kq.gen_matrix("q4k", 31 + m, n, k), kq.gen_x(32 + m, m, k)
        c = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
        try:
            _tune("gemm_few", 2)
            other = gpu_gemm(gpu, "q4k", buf, a, m, n, k)
        finally:
            _tune("gemm_few", 0)
        assert kq.rel_l2(c, _c64("q4k", buf, a, n, k)) <= TOL
        assert np.array_equal(c, other) != taken, (m, n, k)
