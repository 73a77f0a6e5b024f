"""Pins for the CPU oracle (no GPU).  The reference holds no numeric vector for this path - its tests
only inspect PTX text - so the oracle is pinned by what the formats and the mathematics fix:
  * decode A (Q4_K) and C (Q6_K) equal the public GGML block definitions, restated here with GGML's
    own loop structure (different from both oracle restatements);
  * scatter bit maps: flipping one stored bit changes exactly the values, by exactly the amount, that
    a hand-derived bit -> value map says (catches transposed indices, wrong nibble/bit order);
  * closed forms, exactness (fp64 evaluation rounds to the same f32), brute force over byte values;
  * two independently written restatements (numpy, C) and the CPU baseline's third one agree bit for bit;
  * the reference's own structural constants (quantize.rs:34-53 and its tests :2070-2075, :2205-2222).
"""
import os

import numpy as np
import pytest

from oracle import kquant as kq
from oracle.cref import COracle, CpuBaseline

FMTS = ("q4k", "q5k", "q6k")


@pytest.fixture(scope="module")
def co():
    return COracle()


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def f16(v):
    return np.array([v], np.float16).view(np.uint8)


def f32_of_f16(b):
    return np.frombuffer(bytes(b), np.float16).astype(np.float32)[0]


# ---- reference constants (quantize.rs:34-53; tests :2070-2075, :2205-2216, :2360-2369, :2462-2471)
def test_block_constants():
    assert (kq.SUB_BLOCK, kq.SUPER_BLOCK, kq.Q4K_BYTES, kq.Q5K_BYTES, kq.Q6K_BYTES) == (32, 256, 144, 176, 210)
    assert kq.Q4K_BYTES == 2 + 2 + 12 + 128 and kq.Q5K_BYTES == 2 + 2 + 12 + 128 + 32 and kq.Q6K_BYTES == 128 + 64 + 16 + 2


# ---- GGML textbook restatements (public block definitions; GGML's loop structure) -----------
def ggml_get_scale_min_k4(j, q):
    if j < 4:
        return q[j] & 63, q[j + 4] & 63
    return (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4), (q[j + 4] >> 4) | ((q[j] >> 6) << 4)


def ggml_dequantize_row_q4_K(block):
    F = np.float32
    d, dmin = f32_of_f16(block[0:2]), f32_of_f16(block[2:4])
    scales = [int(v) for v in block[4:16]]
    q = [int(v) for v in block[16:144]]
    y, is_, qo = [], 0, 0
    for _ in range(0, 256, 64):
        sc, m = ggml_get_scale_min_k4(is_ + 0, scales)
        d1, m1 = F(d * F(sc)), F(dmin * F(m))
        sc, m = ggml_get_scale_min_k4(is_ + 1, scales)
        d2, m2 = F(d * F(sc)), F(dmin * F(m))
        y += [F(F(d1 * F(q[qo + l] & 0xF)) - m1) for l in range(32)]
        y += [F(F(d2 * F(q[qo + l] >> 4)) - m2) for l in range(32)]
        qo += 32
        is_ += 2
    return np.array(y, np.float32)


def ggml_dequantize_row_q6_K(block):
    F = np.float32
    d = f32_of_f16(block[208:210])
    ql = [int(v) for v in block[0:128]]
    qh = [int(v) for v in block[128:192]]
    sc = [int(v) for v in block[192:208].view(np.int8)]
    y = [F(0)] * 256
    yo = qlo = qho = sco = 0
    for _ in range(0, 256, 128):
        for l in range(32):
            is_ = l // 16
            q1 = ((ql[qlo + l] & 0xF) | (((qh[qho + l] >> 0) & 3) << 4)) - 32
            q2 = ((ql[qlo + l + 32] & 0xF) | (((qh[qho + l] >> 2) & 3) << 4)) - 32
            q3 = ((ql[qlo + l] >> 4) | (((qh[qho + l] >> 4) & 3) << 4)) - 32
            q4 = ((ql[qlo + l + 32] >> 4) | (((qh[qho + l] >> 6) & 3) << 4)) - 32
            y[yo + l + 0] = F(F(d * F(sc[sco + is_ + 0])) * F(q1))
            y[yo + l + 32] = F(F(d * F(sc[sco + is_ + 2])) * F(q2))
            y[yo + l + 64] = F(F(d * F(sc[sco + is_ + 4])) * F(q3))
            y[yo + l + 96] = F(F(d * F(sc[sco + is_ + 6])) * F(q4))
        yo += 128
        qlo += 64
        qho += 32
        sco += 8
    return np.array(y, np.float32)


def test_q4k_is_ggml_q4_K():
    buf = kq.gen_q4k(np.random.default_rng(1), 24).reshape(24, 144)
    got = kq.dequant_q4k(buf.reshape(-1))
    for b in range(24):
        assert np.array_equal(bits(got[b]), bits(ggml_dequantize_row_q4_K(buf[b]))), b


def test_q6k_is_ggml_q6_K():
    buf = kq.gen_q6k(np.random.default_rng(2), 24).reshape(24, 210)
    got = kq.dequant_q6k(buf.reshape(-1))
    for b in range(24):
        assert np.array_equal(bits(got[b]), bits(ggml_dequantize_row_q6_K(buf[b]))), b


# ---- scatter bit maps ------------------------------------------------------------------------
# For a block with d = 1, dmin = 1 and every scale/min field = 1, w = q - 1 (Q4/Q5) or q - 32 (Q6),
# so setting one quant bit raises exactly the mapped value(s) by the mapped power of two.
def _unit_block(fmt):
    blk = np.zeros(kq.SB_BYTES[fmt], np.uint8)
    if fmt == "q6k":
        blk[192:208] = 1
        blk[208:210] = f16(1.0)
        return blk
    blk[0:2] = f16(1.0)
    blk[2:4] = f16(1.0)
    if fmt == "q4k":      # get_scale_min_k4: s_j = m_j = 1 for all eight sub-blocks
        blk[4:8] = 1      # s0..3
        blk[8:12] = 1     # m0..3
        blk[12:16] = 0x11  # s4..7 low nibble, m4..7 high nibble
    else:                 # contiguous 12-bit fields: s = 1, m = 1  ->  0x041 per field
        field = 1 | (1 << 6)
        acc = 0
        for j in range(8):
            acc |= field << (12 * j)
        blk[4:16] = np.frombuffer(acc.to_bytes(12, "little"), np.uint8)
    return blk


def _quant_bit_map(fmt):
    """hand-derived: (byte, bit) -> (value index, increment of the integer quant)"""
    m = {}
    if fmt in ("q4k", "q5k"):
        for B in range(128):           # qs byte B: chunk B//32, low nibble = value 64c + B%32, high = +32
            for b in range(8):
                m[(16 + B, b)] = (64 * (B // 32) + (B % 32) + 32 * (b // 4), 1 << (b % 4))
        if fmt == "q5k":
            for B in range(32):        # qh byte B, bit b: value 8B + b, weight 16
                for b in range(8):
                    m[(144 + B, b)] = (8 * B + b, 16)
    else:
        for B in range(128):           # ql byte B: half B//64, within-half byte p; p<32: groups 0 (low) / 2 (high); p>=32: groups 1 / 3
            h, p = B // 64, B % 64
            for b in range(8):
                g = (1 if p >= 32 else 0) + 2 * (b // 4)
                m[(B, b)] = (128 * h + 32 * g + (p % 32), 1 << (b % 4))
        for B in range(64):            # qh byte B: half B//32, l = B%32; bits 2g, 2g+1 -> group g, weights 16, 32
            h, l = B // 32, B % 32
            for b in range(8):
                m[(128 + B, b)] = (128 * h + 32 * (b // 2) + l, 16 << (b % 2))
    return m


@pytest.mark.parametrize("fmt", FMTS)
def test_scatter_bit_map(fmt, co):
    base_blk = _unit_block(fmt)
    base = kq.DEQUANT[(fmt, 0)](base_blk)[0]
    offset = -32.0 if fmt == "q6k" else -1.0
    assert np.all(base == offset)
    bitmap = _quant_bit_map(fmt)
    n_quant_bits = {"q4k": 128 * 8, "q5k": 160 * 8, "q6k": 192 * 8}[fmt]
    assert len(bitmap) == n_quant_bits
    blocks = np.tile(base_blk, (n_quant_bits, 1))
    keys = sorted(bitmap)
    for row, (byte, bit) in enumerate(keys):
        blocks[row, byte] |= 1 << bit
    w = kq.DEQUANT[(fmt, 0)](blocks.reshape(-1))
    wc = co.dequant(fmt, blocks.reshape(-1), 0)
    assert np.array_equal(bits(w), bits(wc))
    for row, key in enumerate(keys):
        idx, inc = bitmap[key]
        expect = np.full(256, offset, np.float32)
        expect[idx] += inc
        assert np.array_equal(w[row], expect), (fmt, key)


def test_q4k_scale_field_map():
    """every stored scale/min bit of Q4_K moves exactly one (sub-block, field) by a power of two"""
    expect = {}
    for j in range(4):
        for b in range(6):
            expect[(4 + j, b)] = ("s", j, 1 << b)
            expect[(8 + j, b)] = ("m", j, 1 << b)
        for b in (6, 7):
            expect[(4 + j, b)] = ("s", j + 4, 16 << (b - 6))
            expect[(8 + j, b)] = ("m", j + 4, 16 << (b - 6))
        for b in range(4):
            expect[(12 + j, b)] = ("s", j + 4, 1 << b)
            expect[(12 + j, 4 + b)] = ("m", j + 4, 1 << b)
    assert len(expect) == 96
    for (byte, bit), (kind, j, inc) in expect.items():
        sc = np.zeros((1, 12), np.uint8)
        sc[0, byte - 4] = 1 << bit
        s, m = kq.scales_mins_k4(sc)
        want_s, want_m = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
        (want_s if kind == "s" else want_m)[j] = inc
        assert np.array_equal(s[0], want_s) and np.array_equal(m[0], want_m), (byte, bit)


def test_12bit_scale_field_map():
    """Q5_K (and the GEMM-family decodes): bit t of the 96-bit little-endian string belongs to field t//12"""
    for t in range(96):
        sc = np.zeros((1, 12), np.uint8)
        sc[0, t // 8] = 1 << (t % 8)
        s, m = kq.scales_mins_12bit(sc)
        j, r = t // 12, t % 12
        want_s, want_m = np.zeros(8, np.uint8), np.zeros(8, np.uint8)
        (want_s if r < 6 else want_m)[j] = 1 << (r % 6)
        assert np.array_equal(s[0], want_s) and np.array_equal(m[0], want_m), t


def test_q6k_scale_map_and_sign():
    """scale byte 8h + is + 2g governs values 128h + 32g + 16is + 0..15; 0xFF is -1 (decode C), 255 (decode C')"""
    for sidx in range(16):
        blk = np.zeros(210, np.uint8)
        blk[208:210] = f16(1.0)
        blk[192 + sidx] = 0xFF
        w = kq.dequant_q6k(blk)[0]
        h, rem = sidx // 8, sidx % 8
        g, is_ = rem // 2, rem % 2
        lo = 128 * h + 32 * g + 16 * is_
        expect = np.zeros(256, np.float32)
        expect[lo:lo + 16] = 32.0          # (-1) * (0 - 32)
        assert np.array_equal(w, expect), sidx
        wl = kq.dequant_q6k_legacy(blk)[0]
        expect_l = np.zeros(256, np.float32)
        expect_l[16 * sidx:16 * sidx + 16] = 255.0 * -32.0
        assert np.array_equal(wl, expect_l), sidx


# ---- GEMM-family ("legacy", as written) decodes A', B', C' ---------------------------------------
# quantize.rs:445-514 (A'), :727-807 (B'), :1009-1064 (C').  What the cited index arithmetic fixes, derived by hand:
#   A'/B': sub-block j = i // 32 reads its (scale, min) from the 12-bit field j; value i = 32 j + lane reads
#          qs[16 j + lane // 2] = qs[i // 2], low nibble for even i (:488-507); B' adds bit i % 8 of qh[i // 8]
#          at byte 144, weight 16 (:781-795); scale and min are multiplied by rn(1/63) first (:477-482).
#   C'   : 16 sub-blocks of 16; value i reads ql[i // 2] (nibble i & 1), bits 2 (i % 4) of qh[i // 4] at byte 128
#          with weight FOUR (q = ql + 4 qh - 32, :1051-1057), scale = unsigned byte 192 + i // 16.
def _unit_block_legacy(fmt):
    """d = 1 (dmin = 1), every scale field at the value that normalises to exactly 1: w = q - 1 (A', B'), q - 32 (C')"""
    blk = np.zeros(kq.SB_BYTES[fmt], np.uint8)
    if fmt == "q6k":
        blk[192:208] = 1
        blk[208:210] = f16(1.0)
        return blk
    blk[0:2] = f16(1.0)
    blk[2:4] = f16(1.0)
    blk[4:16] = 0xFF          # s_j = m_j = 63, and rn(63 * rn(1/63)) == 1 (asserted below)
    return blk


def _quant_bit_map_legacy(fmt):
    m = {}
    if fmt in ("q4k", "q5k"):
        for B in range(128):           # qs byte B holds values 2B (low nibble) and 2B + 1 (high nibble)
            for b in range(8):
                m[(16 + B, b)] = (2 * B + b // 4, 1 << (b % 4))
        if fmt == "q5k":
            for B in range(32):
                for b in range(8):
                    m[(144 + B, b)] = (8 * B + b, 16)
    else:
        for B in range(128):           # ql byte B: values 2B, 2B + 1
            for b in range(8):
                m[(B, b)] = (2 * B + b // 4, 1 << (b % 4))
        for B in range(64):            # qh byte B: values 4B .. 4B + 3, two bits each, weight 4 (not 16)
            for b in range(8):
                m[(128 + B, b)] = (4 * B + b // 2, 4 << (b % 2))
    return m


def test_inv63_normalises_63_to_one():
    inv63 = np.float32(1.0) / np.float32(63.0)
    assert np.float32(63.0) * inv63 == np.float32(1.0)


@pytest.mark.parametrize("fmt", FMTS)
def test_scatter_bit_map_legacy(fmt, co):
    base_blk = _unit_block_legacy(fmt)
    base = kq.DEQUANT[(fmt, 1)](base_blk)[0]
    offset = -32.0 if fmt == "q6k" else -1.0
    assert np.all(base == offset)
    bitmap = _quant_bit_map_legacy(fmt)
    n_quant_bits = {"q4k": 128 * 8, "q5k": 160 * 8, "q6k": 192 * 8}[fmt]
    assert len(bitmap) == n_quant_bits
    keys = sorted(bitmap)
    blocks = np.tile(base_blk, (n_quant_bits, 1))
    for row, (byte, bit) in enumerate(keys):
        blocks[row, byte] |= 1 << bit
    w = kq.DEQUANT[(fmt, 1)](blocks.reshape(-1))
    assert np.array_equal(bits(w), bits(co.dequant(fmt, blocks.reshape(-1), 1)))
    for row, key in enumerate(keys):
        idx, inc = bitmap[key]
        expect = np.full(256, offset, np.float32)
        expect[idx] += inc
        assert np.array_equal(w[row], expect), (fmt, key)
    # the legacy map is NOT the GEMV-family one: the same one-hot blocks decode differently under policy 0
    w0 = kq.DEQUANT[(fmt, 0)](blocks.reshape(-1))
    assert not np.array_equal(np.argmax(w0 != w0[:, :1], axis=1), np.argmax(w != w[:, :1], axis=1))


@pytest.mark.parametrize("fmt", ("q4k", "q5k"))
def test_legacy_scale_and_min_select_subblock(fmt):
    """A'/B': field j governs values 32 j .. 32 j + 31.  One field at a time: with q = 1 everywhere and dmin = 0,
    w = rn(d * rn(s * rn(1/63))); with q = 0, w = -rn(dmin * rn(m * rn(1/63)))."""
    F = np.float32
    inv63 = F(1.0) / F(63.0)
    d, dmin = F(np.float16(0.0173)), F(np.float16(0.0081))
    for j in range(8):
        for kind in ("s", "m"):
            val = 37 + j
            field = val << (12 * j + (0 if kind == "s" else 6))
            blk = np.zeros(kq.SB_BYTES[fmt], np.uint8)
            blk[0:2] = f16(d)
            blk[2:4] = f16(dmin)
            blk[4:16] = np.frombuffer(field.to_bytes(12, "little"), np.uint8)
            blk[16:144] = 0x11
            w = kq.DEQUANT[(fmt, 1)](blk)[0]
            expect = np.zeros(256, np.float32)
            if kind == "s":
                expect[32 * j:32 * j + 32] = F(F(d * F(F(val) * inv63)) * F(1.0))
            else:
                expect[32 * j:32 * j + 32] = F(F(0.0) - F(dmin * F(F(val) * inv63)))
            assert np.array_equal(bits(w), bits(expect)), (fmt, j, kind)


def test_legacy_q6k_closed_forms():
    """C': all-zero quants -> rn(d * sc) * (-32) with the UNSIGNED scale of sub-block i // 16; qh weighs 4:
    ql = 15 and q2 = 3 give q = 15 + 12 - 32 = -5 (the GEMV-family decode would give 63 - 32 = 31)."""
    F = np.float32
    blk = kq.gen_q6k(np.random.default_rng(77), 8).reshape(8, 210).copy()
    blk[:, :192] = 0
    w = kq.dequant_q6k_legacy(blk.reshape(-1))
    d = np.array([f32_of_f16(b[208:210]) for b in blk], np.float32)
    sc = blk[:, 192:208].astype(np.float32)                     # unsigned
    expect = np.repeat((d[:, None] * sc).astype(F), 16, axis=1) * F(-32.0)
    assert np.array_equal(bits(w), bits(expect))
    blk[:, :192] = 0xFF
    w = kq.dequant_q6k_legacy(blk.reshape(-1))
    assert np.array_equal(bits(w), bits(np.repeat((d[:, None] * sc).astype(F), 16, axis=1) * F(-5.0)))
    assert np.array_equal(bits(kq.dequant_q6k(blk.reshape(-1))[:, :1]),
                          bits((d * blk[:, 192].view(np.int8).astype(F))[:, None] * F(31.0)))


@pytest.mark.parametrize("fmt", ("q4k", "q5k"))
def test_legacy_contraction_ambiguity_is_visible(fmt):
    """A'/B' are inexact: the sequence mul, mul, sub (the definition used here) and the sequence in which the last
    mul and the sub are one fused multiply-add differ on some values, and never by more than one rounding."""
    F = np.float32
    inv63 = F(1.0) / F(63.0)
    blk = kq.GEN[fmt](np.random.default_rng(91), 64).reshape(64, -1)
    w = kq.DEQUANT[(fmt, 1)](blk.reshape(-1))
    d = np.array([f32_of_f16(b[0:2]) for b in blk], F)
    dmin = np.array([f32_of_f16(b[2:4]) for b in blk], F)
    s, m = kq.scales_mins_12bit(blk[:, 4:16])
    ds = np.repeat((d[:, None] * (s.astype(F) * inv63)).astype(F), 32, axis=1)
    dm = np.repeat((dmin[:, None] * (m.astype(F) * inv63)).astype(F), 32, axis=1)
    q = np.empty((64, 256), np.float64)
    q[:, 0::2] = blk[:, 16:144] & 15
    q[:, 1::2] = blk[:, 16:144] >> 4
    if fmt == "q5k":
        q += 16.0 * np.unpackbits(blk[:, 144:176], axis=1, bitorder="little")
    fused = (ds.astype(np.float64) * q - dm.astype(np.float64)).astype(F)     # exact product, one rounding
    differ = bits(fused) != bits(w)
    assert differ.any() and not differ.all()
    ulp = np.spacing(np.maximum(np.abs(w), np.abs(fused)).astype(F))
    assert np.all(np.abs(w.astype(np.float64) - fused.astype(np.float64)) <= 2.0 * ulp.astype(np.float64) + 2.0 * np.spacing(np.abs(ds * q.astype(F)).astype(F)))


# ---- closed forms -----------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", ("q4k", "q5k"))
def test_closed_form_zero_quants(fmt):
    """all quants zero: w = -(dmin * m_j)"""
    rng = np.random.default_rng(5)
    blk = kq.GEN[fmt](rng, 16).reshape(16, -1).copy()
    blk[:, 16:] = 0
    w = kq.DEQUANT[(fmt, 0)](blk.reshape(-1))
    dmin = np.array([f32_of_f16(b[2:4]) for b in blk], np.float32)
    _, m = (kq.scales_mins_k4 if fmt == "q4k" else kq.scales_mins_12bit)(blk[:, 4:16])
    expect = -(dmin[:, None] * m.astype(np.float32))
    assert np.array_equal(w.reshape(16, 8, 32), np.repeat(expect[:, :, None], 32, axis=2))


def test_closed_form_q6k_zero_quants():
    blk = kq.gen_q6k(np.random.default_rng(6), 16).reshape(16, 210).copy()
    blk[:, :192] = 0
    w = kq.dequant_q6k(blk.reshape(-1))
    d = np.array([f32_of_f16(b[208:210]) for b in blk], np.float32)
    sc = blk[:, 192:208].view(np.int8).astype(np.float32)
    i = np.arange(256)
    sidx = 8 * (i // 128) + (i % 32) // 16 + 2 * ((i % 128) // 32)
    assert np.array_equal(w, (d[:, None] * sc[:, sidx]) * np.float32(-32.0))


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("policy", (0, 1))
def test_exactness_and_two_restatements(fmt, policy, co):
    """canonical decodes: the fp64 evaluation rounded once equals the f32 evaluation; both families:
    numpy and C restatements agree bit for bit (incl. forced subnormal / zero / max f16 fields)"""
    rng = np.random.default_rng(11)
    blk = kq.GEN[fmt](rng, 4000).reshape(4000, -1).copy()
    offs = (208,) if fmt == "q6k" else (0, 2)
    for i, hbits in enumerate((0x0000, 0x0001, 0x03FF, 0x0400, 0x7BFF, 0x8001, 0xFBFF)):
        for o in offs:
            blk[i, o:o + 2] = np.array([hbits], np.uint16).view(np.uint8)
    w = kq.DEQUANT[(fmt, policy)](blk.reshape(-1))
    assert np.array_equal(bits(w), bits(co.dequant(fmt, blk.reshape(-1), policy)))
    if policy == 0:
        if fmt == "q6k":
            d = blk[:, 208:210].copy().view(np.float16).astype(np.float64)
            sc = blk[:, 192:208].view(np.int8).astype(np.float64)
            i = np.arange(256)
            h, g, l = i // 128, (i % 128) // 32, i % 32
            sidx = 8 * h + l // 16 + 2 * g
            nib = (blk[:, 64 * h + l + 32 * (g & 1)].astype(np.int64) >> (4 * (g >> 1))) & 15
            q2 = (blk[:, 128 + 32 * h + l].astype(np.int64) >> (2 * g)) & 3
            exact = d * sc[:, sidx] * ((nib | (q2 << 4)) - 32).astype(np.float64)
        else:
            d = blk[:, 0:2].copy().view(np.float16).astype(np.float64)
            dmin = blk[:, 2:4].copy().view(np.float16).astype(np.float64)
            s, m = (kq.scales_mins_k4 if fmt == "q4k" else kq.scales_mins_12bit)(blk[:, 4:16])
            ql = kq._nibbles_chunked(blk[:, 16:144]).astype(np.float64)
            if fmt == "q5k":
                ql = ql + 16.0 * np.unpackbits(blk[:, 144:176], axis=1, bitorder="little")
            exact = np.repeat(d * s, 32, axis=1) * ql - np.repeat(dmin * m, 32, axis=1)
        assert np.array_equal(bits(exact.astype(np.float32)), bits(w))


@pytest.mark.parametrize("fmt", FMTS)
def test_byte_brute_force(fmt, co):
    """every value of one byte position x a spread of positions: numpy == C == CPU-baseline decode"""
    cb = CpuBaseline()
    base = kq.GEN[fmt](np.random.default_rng(21), 1)
    rng = np.random.default_rng(22)
    for pos in rng.choice(kq.SB_BYTES[fmt], 16, replace=False):
        blocks = np.tile(base, (256, 1))
        blocks[:, pos] = np.arange(256, dtype=np.uint8)
        if fmt == "q6k" and pos == 209 or fmt != "q6k" and pos in (1, 3):
            blocks[:, pos] &= 0x7B      # keep the f16 finite
        w = kq.DEQUANT[(fmt, 0)](blocks.reshape(-1))
        assert np.array_equal(bits(w), bits(co.dequant(fmt, blocks.reshape(-1), 0))), pos
        for r in (0, 77, 255):
            assert np.array_equal(bits(cb.decode_block(fmt, blocks[r])), bits(w[r])), (pos, r)


# ---- products ----------------------------------------------------------------------------------
@pytest.mark.parametrize("fmt", FMTS)
def test_gemv_brute_force_tiny(fmt, co):
    n, k = 3, 512
    buf, x = kq.gen_matrix(fmt, 31, n, k), kq.gen_x(32, k)
    w = kq.dequant_matrix(fmt, buf, n, k)
    y = kq.gemv_fp64(w, x)
    brute = [sum(float(w[r, i]) * float(x[i]) for i in range(k)) for r in range(n)]
    assert np.allclose(y, brute, rtol=1e-13, atol=0)
    assert np.allclose(co.gemv_fp64(fmt, buf, x, k, n), brute, rtol=1e-13, atol=0)
    a = kq.gen_x(33, 2, k)
    c = kq.gemm_fp64(a, w)
    assert c.shape == (2, n) and np.allclose(c[1], kq.gemv_fp64(w, a[1]), rtol=1e-13)
    assert np.allclose(co.gemm_fp64(fmt, buf, a, 2, n, k), c, rtol=1e-13)


@pytest.mark.parametrize("fmt", FMTS)
def test_reference_order_emulation(fmt, co):
    """the lane/summation-order emulation: numpy and C agree, and sit at f32 rounding distance from fp64"""
    n, k = 40, 2048
    buf, x = kq.gen_matrix(fmt, 41, n, k), kq.gen_x(42, k)
    w = kq.dequant_matrix(fmt, buf, n, k)
    a = kq.gemv_ref_order_fp32(w, x)
    b = co.gemv_ref_order_f32(fmt, buf, x, k, n)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
    assert 0 < kq.rel_l2(a, kq.gemv_fp64(w, x)) < 1e-6


def _q6k_all_ones(n_sb):
    """Q6_K super-blocks whose 256 weights are all 1.0: d = 1 (f16 0x3C00), every scale 1, every quant 33
    (low nibble 1 in ql, two-bit field 2 in qh), so w = d * sc * (q - 32) = 1."""
    b = np.zeros((n_sb, 210), np.uint8)
    b[:, :128] = 0x11
    b[:, 128:192] = 0xAA
    b[:, 192:208] = 1
    b[:, 208:210] = [0x00, 0x3C]
    return b.reshape(-1)


def _sum_in_order(x, owner, chain, tree):
    """f32 sum of x (one super-block, all weights 1) for a lane ownership, a chain direction and a tree: a
    deliberately general helper, used only to show that OTHER orders miss the hand-worked values below."""
    f = np.float32
    acc = []
    for t in range(32):
        p = f(0)
        for j in chain:
            p = f(p + f(x[owner(t, j)]))
        acc.append(p)
    for step in tree:
        # steps falling from 16: the shuffle-down tree (lane t takes lane t + step); rising from 1: neighbours first
        for t in (range(step) if tree[0] == 16 else range(0, 32, 2 * step)):
            acc[t] = f(acc[t] + acc[t + step])
    return float(acc[0])


def test_reference_order_hand_worked(co):
    """The yardstick of "no worse than the reference's own f32 result", pinned by cases worked by hand from
    quantize.rs:1412, 1482-1518 (lane t of 32 owns values t + 32 j; p = 0, p = fma(x, w, p) for j = 0..7;
    acc += p per super-block; then acc[i] += acc[i + 16], + 8, + 4, + 2, + 1; lane 0 is the result).

    All weights are 1 and x holds a few powers of two; B = 2^24, where f32 has spacing 2 (B + 1 rounds to B,
    1 - B is exact).  Values of x that are not zero, by index i = t + 32 j:
        i = 0: 1    i = 32: B    i = 64: -B      lane 0:  (1 + B) - B = B - B = 0          (the 1 is lost)
        i = 8: 1                                 lane 8:  1
        i = 4: B    i = 20: 1    i = 12: -B      lanes 4, 20, 12: B, 1, -B
        i = 2: 0.5  i = 1: 0.25                  lanes 2, 1
    tree, step 16:  a0 = p0 + p16 = 0;  a8 = p8 + p24 = 1;  a4 = p4 + p20 = B + 1 = B (lost);  a12 = -B
          step 8:   a0 = 0 + 1 = 1;  a4 = B - B = 0;  step 4: a0 = 1 + 0 = 1;  step 2: a0 = 1 + 0.5;  step 1: + 0.25
    so y = 1.75, where the exact sum is 3.75.  Other orders give other numbers: a chain from j = 7 down keeps lane 0's
    1 (2.75); a tree of neighbours first (1, 2, 4, 8, 16) gives 2; lanes owning 8 t .. 8 t + 7 give 5."""
    B = np.float32(2.0 ** 24)
    x = np.zeros(256, np.float32)
    for i, v in ((0, 1), (32, B), (64, -B), (8, 1), (4, B), (20, 1), (12, -B), (2, 0.5), (1, 0.25)):
        x[i] = v
    assert float(x.astype(np.float64).sum()) == 3.75
    w = np.ones((1, 256), np.float32)
    assert kq.gemv_ref_order_fp32(w, x)[0] == np.float32(1.75)
    blocks = _q6k_all_ones(1)
    assert np.all(kq.dequant_matrix("q6k", blocks, 1, 256) == 1.0)
    assert co.gemv_ref_order_f32("q6k", blocks, x, 256, 1)[0] == np.float32(1.75)
    # the case tells the orders apart
    strided, contiguous = (lambda t, j: t + 32 * j), (lambda t, j: 8 * t + j)
    down_tree, up_tree = (16, 8, 4, 2, 1), (1, 2, 4, 8, 16)
    assert _sum_in_order(x, strided, range(8), down_tree) == 1.75
    assert _sum_in_order(x, strided, range(7, -1, -1), down_tree) == 2.75
    assert _sum_in_order(x, strided, range(8), up_tree) == 2.0
    assert _sum_in_order(x, contiguous, range(8), down_tree) == 5.0

    # Two super-blocks: the partial sum of a super-block is formed on its own and then added (quantize.rs:1412, 1486).
    # Lane 0: super-block 0 holds B; super-block 1 holds 1 (j = 0) and 1 (j = 1): p = 2, acc = B + 2 exactly.  Adding
    # the values to acc one by one would lose both: B + 1 = B, B + 1 = B.
    x2 = np.zeros(512, np.float32)
    x2[0], x2[256], x2[256 + 32] = B, 1, 1
    want = np.float32(2.0 ** 24 + 2)
    assert kq.gemv_ref_order_fp32(np.ones((1, 512), np.float32), x2)[0] == want
    assert co.gemv_ref_order_f32("q6k", _q6k_all_ones(2), x2, 512, 1)[0] == want


def test_row_layout():
    """row n starts at byte n * (k/256) * SB (quantize.rs:1219-1224)"""
    n, k = 5, 768
    for fmt in FMTS:
        buf = kq.gen_matrix(fmt, 51, n, k)
        w = kq.dequant_matrix(fmt, buf, n, k)
        sb = kq.SB_BYTES[fmt]
        row3 = kq.DEQUANT[(fmt, 0)](buf[3 * 3 * sb:4 * 3 * sb]).reshape(-1)
        assert np.array_equal(w[3], row3)
    with pytest.raises(ValueError):
        kq.dequant_matrix("q4k", np.zeros(144, np.uint8), 1, 100)


def test_golden_fixture_matches_oracles(co):
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "kquant_golden.npz"))
    for fmt in FMTS:
        for policy in (0, 1):
            want = z[f"{fmt}_w{policy}_bits"]
            assert np.array_equal(bits(kq.DEQUANT[(fmt, policy)](z[f"{fmt}_blocks"])).reshape(-1), want)
            assert np.array_equal(bits(co.dequant(fmt, z[f"{fmt}_blocks"], policy)).reshape(-1), want)
        w = kq.dequant_matrix(fmt, z[f"{fmt}_gemv_w"], 3, 512)
        assert np.allclose(kq.gemv_fp64(w, z[f"{fmt}_gemv_x"]), z[f"{fmt}_gemv_y64"], rtol=1e-14)


def test_cpu_baseline_matches_fp64():
    cb = CpuBaseline()
    for fmt in FMTS:
        n, k = 4100, 1024          # >= 4096 rows takes the threaded path
        buf, x = kq.gen_matrix(fmt, 61, n, k), kq.gen_x(62, k)
        w = kq.dequant_matrix(fmt, buf, n, k)
        y64 = kq.gemv_fp64(w, x)
        y, _ = cb.dequant_matvec(fmt, buf, x, k, n, threads=4)
        assert kq.rel_l2(y, y64) < 1e-6
        y2, _ = cb.matvec_f32(w, x, threads=4)
        assert np.array_equal(y.view(np.uint32), y2.view(np.uint32))
