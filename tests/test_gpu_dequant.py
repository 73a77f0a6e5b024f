"""GPU parity, dequantisation: every f32 weight bit-exact with the oracle (all three formats, both
decode families), through the C ABI."""
import numpy as np
import pytest

from oracle import kquant as kq
from tests.kq_helpers import SB, gpu_dequant

pytestmark = pytest.mark.gpu

FMTS = ("q4k", "q5k", "q6k")
D_OFF = {"q4k": (0, 2), "q5k": (0, 2), "q6k": (208,)}


def _bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def _special_blocks(fmt: str, rng) -> np.ndarray:
    """Blocks whose f16 fields are forced through zero, subnormals, the smallest/largest normals."""
    specials = np.array([0x0000, 0x0001, 0x0002, 0x03FF, 0x0400, 0x0401, 0x3C00, 0x7BFF, 0x8001, 0xBC00, 0x2E66],
                        np.uint16)
    blk = kq.GEN[fmt](rng, specials.size * specials.size).reshape(-1, SB[fmt]).copy()
    i = 0
    for a in specials:
        for b in specials:
            offs = D_OFF[fmt]
            blk[i, offs[0]:offs[0] + 2] = np.array([a], np.uint16).view(np.uint8)
            if len(offs) > 1:
                blk[i, offs[1]:offs[1] + 2] = np.array([b], np.uint16).view(np.uint8)
            i += 1
    return blk.reshape(-1)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("policy", (0, 1))
def test_dequant_bit_exact_random(gpu, fmt, policy):
    n_sb = 120_000 if policy == 0 else 20_000
    buf = kq.GEN[fmt](np.random.default_rng(100 + policy), n_sb)
    got = gpu_dequant(gpu, fmt, buf, policy)
    want = kq.DEQUANT[(fmt, policy)](buf)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("policy", (0, 1))
def test_dequant_bit_exact_special_f16(gpu, fmt, policy):
    buf = _special_blocks(fmt, np.random.default_rng(7))
    got = gpu_dequant(gpu, fmt, buf, policy)
    want = kq.DEQUANT[(fmt, policy)](buf)
    assert np.array_equal(_bits(got), _bits(want))


@pytest.mark.parametrize("fmt", FMTS)
def test_dequant_all_byte_values(gpu, fmt):
    """every byte value at every byte position of one block, the rest fixed."""
    base = kq.GEN[fmt](np.random.default_rng(3), 1)
    blocks = np.tile(base, (256, 1))
    rng = np.random.default_rng(4)
    for pos in rng.choice(SB[fmt], 24, replace=False):
        b = blocks.copy()
        b[:, pos] = np.arange(256, dtype=np.uint8)
        got = gpu_dequant(gpu, fmt, b.reshape(-1), 0)
        assert np.array_equal(_bits(got), _bits(kq.DEQUANT[(fmt, 0)](b.reshape(-1)))), pos


@pytest.mark.parametrize("fmt", FMTS)
def test_dequant_misaligned_pointer(gpu, fmt):
    """a weight pointer that is only byte aligned takes the byte-load kernel; same bits."""
    buf = kq.GEN[fmt](np.random.default_rng(11), 300)
    want = kq.DEQUANT[(fmt, 0)](buf)
    for off in (1, 2, 6):
        assert np.array_equal(_bits(gpu_dequant(gpu, fmt, buf, 0, w_offset=off)), _bits(want)), off


def test_dequant_golden_fixture(gpu):
    """the committed fixture (tests/golden/kquant_golden.npz): blocks and expected f32 bit patterns."""
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "kquant_golden.npz"))
    for fmt in FMTS:
        for policy in (0, 1):
            got = gpu_dequant(gpu, fmt, z[f"{fmt}_blocks"], policy)
            assert np.array_equal(_bits(got), z[f"{fmt}_w{policy}_bits"].reshape(got.shape)), (fmt, policy)


def test_dequant_empty_and_bad_policy(gpu):
    import trueno_amd as t
    from trueno_amd import kernels as K
    ctx, stream = gpu
    out = t.GpuBuffer(ctx, 256, np.float32)
    w = t.GpuBuffer(ctx, 144, np.uint8)
    K.dequant_f32("q4k", stream, out, w, 0, 0)  # no-op
    with pytest.raises(t.GpuError):
        K.dequant_f32("q4k", stream, out, w, 1, 2)
