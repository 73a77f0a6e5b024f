"""CPU oracle for the k-quant dequantize-and-multiply path (TEST INFRASTRUCTURE ONLY).

This module is a numpy restatement of the arithmetic that trueno-gpu's PTX builder
describes for its fused k-quant kernels.  It exists to check the HIP kernels; nothing
in the product path may import it (only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py do).

Reference lines followed (all under trueno-gpu/src/kernels/quantize.rs):
  decode A  Q4_K, GEMV family   :1237-1483   (GGML dequantize_row_q4_K layout)
  decode B  Q5_K, GEMV family   :1589-1693   (reference-specific layout, NOT GGML)
  decode C  Q6_K, GEMV family   :1806-1934   (GGML dequantize_row_q6_K layout)
  decode A' Q4_K, GEMM family   :445-514     (12-bit scale fields, /63, sequential nibbles)
  decode B' Q5_K, GEMM family   :727-807
  decode C' Q6_K, GEMM family   :1009-1064   (unsigned scales, ql + 4*qh)
  GEMV summation order          :1412-1518   (32 lanes, fma per value, shfl.down tree)
  block constants               :34-53

How each function is pinned (the reference holds no numeric test of this path):
  dequant_q4k / dequant_q6k : equal to the public GGML block definitions restated
      independently in tests/test_oracle_pins.py (different loop structure), plus
      one-hot bit maps, closed forms, byte brute force, and the C restatement
      oracle/kquant_ref.c written separately from the same reference lines.
  dequant_q5k               : only the builder calls define it (no GGML equivalent).  Pinned by the
      scatter map of all 1408 stored bits derived by hand from the cited index arithmetic, the
      12-bit field map, closed forms, exactness (fp64-then-round == f32) and the C restatement.
  dequant_q4k/q5k/q6k_legacy: only the builder calls define them.  Pinned by hand-derived scatter
      maps of every quant bit (sequential nibbles qs[i//2]; B' fifth bit i%8 of qh[i//8]; C'
      ql[i//2], qh[i//4] with weight 4, unsigned scale i//16), one-field-at-a-time scale/min
      selection, closed forms (zero quants, all-ones quants), the visible difference between the
      uncontracted sequence (the definition here) and a fused multiply-subtract, and the C
      restatement.  Each of these fails under a swapped nibble, a wrong weight, a wrong scale
      packing or a signed/unsigned slip.  No reference-held vector exists for any decode, so
      nothing here is checked against a running reference.
  gemv_fp64 / gemm_fp64     : closed form (an fp64 dot product), brute force on tiny shapes.
  gemv_ref_order_fp32       : emulation of the reference's lane/summation order; used only
      to compare error magnitudes, never for bit parity.

All decode arithmetic is IEEE binary32, one rounding per PTX instruction
(mul.f32 / sub.f32 print no rounding modifier = .rn, ptx/builder.rs:1888-1913).
"""
from __future__ import annotations

import numpy as np

# quantize.rs:34-53
SUB_BLOCK = 32
SUPER_BLOCK = 256
Q4K_BYTES = 144
Q5K_BYTES = 176
Q6K_BYTES = 210
SB_BYTES = {"q4k": Q4K_BYTES, "q5k": Q5K_BYTES, "q6k": Q6K_BYTES}

F32 = np.float32


def _f16_at(blocks: np.ndarray, off: int) -> np.ndarray:
    """f16 little-endian at byte `off` of every block -> f32 (cvt.f32.f16 is exact)."""
    raw = blocks[:, off].astype(np.uint16) | (blocks[:, off + 1].astype(np.uint16) << 8)
    return raw.view(np.float16).astype(F32)


def _as_blocks(buf, nbytes: int) -> np.ndarray:
    a = np.ascontiguousarray(np.asarray(buf, dtype=np.uint8)).reshape(-1)
    if a.size % nbytes:
        raise ValueError(f"buffer of {a.size} bytes is not a multiple of {nbytes}")
    return a.reshape(-1, nbytes)


# --------------------------------------------------------------------------------------
# scale / min unpacking
# --------------------------------------------------------------------------------------
def scales_mins_k4(sc: np.ndarray):
    """get_scale_min_k4 packing of eight 6-bit (scale, min) pairs in 12 bytes.
    quantize.rs:1306-1385.  sc: uint8 [n,12] -> (s, m) uint8 [n,8]."""
    sc = sc.astype(np.uint8)
    s = np.empty((sc.shape[0], 8), np.uint8)
    m = np.empty((sc.shape[0], 8), np.uint8)
    for j in range(4):
        s[:, j] = sc[:, j] & 63
        m[:, j] = sc[:, j + 4] & 63
    for j in range(4, 8):
        s[:, j] = (sc[:, j + 4] & 0xF) | ((sc[:, j - 4] >> 6) << 4)
        m[:, j] = (sc[:, j + 4] >> 4) | ((sc[:, j] >> 6) << 4)
    return s, m


def scales_mins_12bit(sc: np.ndarray):
    """Eight contiguous little-endian 12-bit fields (6-bit scale low, 6-bit min high).
    quantize.rs:1607-1635 (also :445-475, :727-750).  sc: uint8 [n,12] -> (s, m) [n,8]."""
    sc = sc.astype(np.uint32)
    s = np.empty((sc.shape[0], 8), np.uint8)
    m = np.empty((sc.shape[0], 8), np.uint8)
    for j in range(8):
        bit = 12 * j
        b, sh = bit // 8, bit % 8
        t = (sc[:, b] | (sc[:, b + 1] << 8)) >> sh
        s[:, j] = t & 63
        m[:, j] = (t >> 6) & 63
    return s, m


# --------------------------------------------------------------------------------------
# canonical (GEMV-family) decodes
# --------------------------------------------------------------------------------------
def _nibbles_chunked(qs: np.ndarray) -> np.ndarray:
    """qs uint8 [n,128] -> 4-bit quants [n,256] in the 64-value-chunk order:
    value i lives in byte 32*(i//64) + i%32, low nibble if i%64 < 32 (quantize.rs:1443-1466)."""
    n = qs.shape[0]
    c = qs.reshape(n, 4, 32)
    out = np.empty((n, 4, 2, 32), np.uint8)
    out[:, :, 0, :] = c & 0xF
    out[:, :, 1, :] = c >> 4
    return out.reshape(n, 256)


def dequant_q4k(buf) -> np.ndarray:
    """Decode A.  Returns f32 [n_sb, 256].  w = (d*s_j)*q - (dmin*m_j)  (quantize.rs:1388-1403, 1468-1471)."""
    blk = _as_blocks(buf, Q4K_BYTES)
    d = _f16_at(blk, 0)
    dmin = _f16_at(blk, 2)
    s, m = scales_mins_k4(blk[:, 4:16])
    ds = d[:, None] * s.astype(F32)            # mul.f32
    dm = dmin[:, None] * m.astype(F32)         # mul.f32
    q = _nibbles_chunked(blk[:, 16:144]).astype(F32)
    ds_v = np.repeat(ds, 32, axis=1)
    dm_v = np.repeat(dm, 32, axis=1)
    scaled = ds_v * q                          # mul.f32
    return (scaled - dm_v).astype(F32)         # sub.f32


def dequant_q5k(buf) -> np.ndarray:
    """Decode B.  Block: d@0 dmin@2 sc[12]@4 qs[128]@16 qh[32]@144.
    q = ql + 16*qh_bit,  qh_bit(i) = (qh[i//8] >> (i%8)) & 1  (quantize.rs:1659-1675);
    w = ((d*s_j)*q) - (dmin*m_j)  (:1677-1682)."""
    blk = _as_blocks(buf, Q5K_BYTES)
    d = _f16_at(blk, 0)
    dmin = _f16_at(blk, 2)
    s, m = scales_mins_12bit(blk[:, 4:16])
    ql = _nibbles_chunked(blk[:, 16:144]).astype(np.uint32)
    qh = np.unpackbits(blk[:, 144:176], axis=1, bitorder="little").astype(np.uint32)  # bit i of 256
    q = (ql + 16 * qh).astype(F32)
    ds_v = np.repeat(d[:, None] * s.astype(F32), 32, axis=1)
    dm_v = np.repeat(dmin[:, None] * m.astype(F32), 32, axis=1)
    return ((ds_v * q) - dm_v).astype(F32)


def dequant_q5k_ggml(buf) -> np.ndarray:
    """GGML's own Q5_K block (public format: block_q5_K = d, dmin, scales[12], qh[32], qs[128]; dequantize_row_q5_K):
    scales/mins packed as in Q4_K (get_scale_min_k4); value i = 32 j + l has the nibble of qs[32 (i//64) + l] (low for
    even j) and its fifth bit in bit j of qh[l];  w = (d*sc_j)*q - dmin*m_j.  NOT the reference's Q5_K layout - this
    is what a GGUF file holds; q5k_ggml_to_reference() turns one into the other."""
    blk = _as_blocks(buf, Q5K_BYTES)
    d = _f16_at(blk, 0)
    dmin = _f16_at(blk, 2)
    s, m = scales_mins_k4(blk[:, 4:16])
    qh = blk[:, 16:48].astype(np.uint32)
    ql = _nibbles_chunked(blk[:, 48:176]).astype(np.uint32)
    i = np.arange(256)
    hb = (qh[:, i % 32] >> (i // 32)) & 1
    q = (ql + 16 * hb).astype(F32)
    ds_v = np.repeat(d[:, None] * s.astype(F32), 32, axis=1)
    dm_v = np.repeat(dmin[:, None] * m.astype(F32), 32, axis=1)
    return ((ds_v * q) - dm_v).astype(F32)


def q5k_ggml_to_reference(buf) -> np.ndarray:
    """Re-pack GGML Q5_K blocks into the layout decode B reads (quantize.rs:1589-1693): header kept, the eight
    (scale, min) pairs as contiguous 12-bit fields, qs moved to offset 16, the fifth bits re-ordered so that value i
    is bit i%8 of qh[i//8] at offset 144.  dequant_q5k(result) == dequant_q5k_ggml(input), bit for bit."""
    blk = _as_blocks(buf, Q5K_BYTES)
    out = np.zeros_like(blk)
    out[:, 0:4] = blk[:, 0:4]
    s, m = scales_mins_k4(blk[:, 4:16])
    fields = (s.astype(np.uint64) | (m.astype(np.uint64) << np.uint64(6)))          # 12 bits each
    bits = np.zeros((blk.shape[0], 96), np.uint8)
    for j in range(8):
        for r in range(12):
            bits[:, 12 * j + r] = (fields[:, j] >> np.uint64(r)) & np.uint64(1)
    out[:, 4:16] = np.packbits(bits, axis=1, bitorder="little")
    out[:, 16:144] = blk[:, 48:176]
    i = np.arange(256)
    hb = ((blk[:, 16:48][:, i % 32] >> (i // 32)) & 1).astype(np.uint8)
    out[:, 144:176] = np.packbits(hb, axis=1, bitorder="little")
    return out.reshape(-1)


def dequant_q6k(buf) -> np.ndarray:
    """Decode C.  Block: ql[128]@0 qh[64]@128 sc[16] int8 @192 d@208.
    value i: h=i//128, p=i%128, g=p//32, l=p%32; scale sc[8h + l//16 + 2g];
    nibble of ql[64h + l + 32*(g&1)], high iff g>=2; q2=(qh[32h+l]>>(2g))&3;
    w = (d*sc) * ((nib | q2<<4) - 32)   (quantize.rs:1829-1923)."""
    blk = _as_blocks(buf, Q6K_BYTES)
    n = blk.shape[0]
    d = _f16_at(blk, 208)
    sc = blk[:, 192:208].view(np.int8).astype(F32)      # u8 - 256*(u8>>7) in f32 == sign extension
    i = np.arange(256)
    h, p = i // 128, i % 128
    g, l = p // 32, p % 32
    sidx = 8 * h + l // 16 + 2 * g
    qlb = blk[:, 64 * h + l + 32 * (g & 1)].astype(np.uint32)
    nib = (qlb >> (4 * (g >> 1))) & 0xF
    q2 = (blk[:, 128 + 32 * h + l].astype(np.uint32) >> (2 * g)) & 3
    comb = (nib | (q2 << 4)).astype(F32)
    qs = comb - F32(32.0)                                # sub.f32
    dsc = d[:, None] * sc[:, sidx]                       # mul.f32
    out = dsc * qs                                       # mul.f32
    assert out.shape == (n, 256)
    return out.astype(F32)


# --------------------------------------------------------------------------------------
# legacy (GEMM-family, as written) decodes.  Uncontracted mul/sub sequence.
# --------------------------------------------------------------------------------------
INV63 = F32(1.0) / F32(63.0)   # mov_f32_imm(1.0 / 63.0), quantize.rs:480


def _nibbles_sequential(qs: np.ndarray) -> np.ndarray:
    """value i -> qs[i//2], low nibble for even i (quantize.rs:488-507)."""
    n = qs.shape[0]
    out = np.empty((n, 128, 2), np.uint8)
    out[:, :, 0] = qs & 0xF
    out[:, :, 1] = qs >> 4
    return out.reshape(n, 256)


def dequant_q4k_legacy(buf) -> np.ndarray:
    """Decode A'.  w = ((d*(s*inv63))*q) - (dmin*(m*inv63))  (quantize.rs:477-514)."""
    blk = _as_blocks(buf, Q4K_BYTES)
    d = _f16_at(blk, 0)
    dmin = _f16_at(blk, 2)
    s, m = scales_mins_12bit(blk[:, 4:16])
    sn = s.astype(F32) * INV63
    mn = m.astype(F32) * INV63
    q = _nibbles_sequential(blk[:, 16:144]).astype(F32)
    ds_v = np.repeat(d[:, None] * sn, 32, axis=1)
    dm_v = np.repeat(dmin[:, None] * mn, 32, axis=1)
    return ((ds_v * q) - dm_v).astype(F32)


def dequant_q5k_legacy(buf) -> np.ndarray:
    """Decode B'.  A' plus the fifth bit (qh[i//8]>>(i%8))&1 at offset 144  (quantize.rs:727-807)."""
    blk = _as_blocks(buf, Q5K_BYTES)
    d = _f16_at(blk, 0)
    dmin = _f16_at(blk, 2)
    s, m = scales_mins_12bit(blk[:, 4:16])
    sn = s.astype(F32) * INV63
    mn = m.astype(F32) * INV63
    ql = _nibbles_sequential(blk[:, 16:144]).astype(np.uint32)
    qh = np.unpackbits(blk[:, 144:176], axis=1, bitorder="little").astype(np.uint32)
    q = (ql + 16 * qh).astype(F32)
    ds_v = np.repeat(d[:, None] * sn, 32, axis=1)
    dm_v = np.repeat(dmin[:, None] * mn, 32, axis=1)
    return ((ds_v * q) - dm_v).astype(F32)


def dequant_q6k_legacy(buf) -> np.ndarray:
    """Decode C'.  scale = UNSIGNED sc[i//16]; ql[i//2] nibble i&1; q2=(qh[i//4]>>2(i%4))&3;
    q = ql + 4*q2 - 32; w = (d*sc)*q   (quantize.rs:1009-1064)."""
    blk = _as_blocks(buf, Q6K_BYTES)
    d = _f16_at(blk, 208)
    sc = blk[:, 192:208].astype(F32)
    i = np.arange(256)
    ql = (blk[:, i // 2].astype(np.uint32) >> (4 * (i & 1))) & 0xF
    q2 = (blk[:, 128 + i // 4].astype(np.uint32) >> (2 * (i % 4))) & 3
    qf = (ql + 4 * q2).astype(F32) - F32(32.0)
    dsc = d[:, None] * sc[:, i // 16]
    return (dsc * qf).astype(F32)


Q4K_SIMPLE_BLOCK = 32
Q4K_SIMPLE_BYTES = 18


def dequant_q4k_simplified(buf) -> np.ndarray:
    """Legacy "simplified" Q4_K of q4k_gemm_fused (quantize.rs:41, 151-336): blocks of 32 values in 18
    bytes - f16 scale at 0 (:237-241), 16 bytes of nibbles at 2 (:250-254); value i sits in byte i/2,
    low nibble for even i (:245-262); w = scale * q, no min term (:264-267).  Returns [n_blocks, 32] f32."""
    b = _as_blocks(buf, Q4K_SIMPLE_BYTES)
    scale = _f16_at(b, 0).astype(np.float32)
    qs = b[:, 2:18].astype(np.uint32)
    q = np.empty((b.shape[0], 32), np.uint32)
    q[:, 0::2] = qs & 15
    q[:, 1::2] = qs >> 4
    return (scale[:, None] * q.astype(np.float32)).astype(np.float32)


def dequant_matrix_simplified(buf, n: int, k: int) -> np.ndarray:
    """n rows x (k/32) blocks of 18 bytes, row-major (quantize.rs:225-231) -> f32 [n, k]."""
    if k % Q4K_SIMPLE_BLOCK:
        raise ValueError("k must be a multiple of 32")
    w = dequant_q4k_simplified(buf)
    if w.shape[0] != n * (k // Q4K_SIMPLE_BLOCK):
        raise ValueError("buffer size does not match n x k")
    return w.reshape(n, k)


DEQUANT = {
    ("q4k", 0): dequant_q4k, ("q5k", 0): dequant_q5k, ("q6k", 0): dequant_q6k,
    ("q4k", 1): dequant_q4k_legacy, ("q5k", 1): dequant_q5k_legacy, ("q6k", 1): dequant_q6k_legacy,
}


def dequant_matrix(fmt: str, buf, n: int, k: int, policy: int = 0) -> np.ndarray:
    """Row-major matrix of n rows x (k/256) super-blocks -> f32 [n, k]
    (row n starts at byte n*(k/256)*SB, quantize.rs:1219-1224)."""
    if k % SUPER_BLOCK:
        raise ValueError("k must be a multiple of 256")
    w = DEQUANT[(fmt, policy)](buf)
    if w.shape[0] != n * (k // SUPER_BLOCK):
        raise ValueError("buffer size does not match n x k")
    return w.reshape(n, k)


# --------------------------------------------------------------------------------------
# products
# --------------------------------------------------------------------------------------
def gemv_fp64(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    """y = W x in fp64 from the f32 dequantised weights (the tolerance reference)."""
    return w.astype(np.float64) @ np.asarray(x, np.float32).astype(np.float64)


def gemm_fp64(a: np.ndarray, w: np.ndarray) -> np.ndarray:
    """C[m,n] = A[m,k] . W[n,k]^T in fp64; C row-major c[row*n+col] (quantize.rs:568-574)."""
    return np.asarray(a, np.float32).astype(np.float64) @ w.astype(np.float64).T


def gemv_ref_order_fp32(w: np.ndarray, x: np.ndarray) -> np.ndarray:
    """f32 result in the reference's summation order (quantize.rs:1412, 1482-1518):
    lane t of 32 owns values t+32j; per super-block p=0, p=fma(x,w,p) for j=0..7; acc+=p;
    then acc_i += acc_{i+16}, +8, +4, +2, +1; lane 0 is y[n].
    fma is evaluated as an fp64 product (exact) plus fp64 add rounded to f32; the rare
    double-rounding difference from a true fma does not matter for an error comparison."""
    n, k = w.shape
    x = np.asarray(x, np.float32)
    nsb = k // SUPER_BLOCK
    wv = w.reshape(n, nsb, 8, 32).astype(np.float64)
    xv = x.reshape(nsb, 8, 32).astype(np.float64)
    acc = np.zeros((n, 32), F32)
    for sb in range(nsb):
        p = np.zeros((n, 32), F32)
        for j in range(8):
            p = (wv[:, sb, j, :] * xv[sb, j, :] + p.astype(np.float64)).astype(F32)
        acc = (acc + p).astype(F32)
    for step in (16, 8, 4, 2, 1):
        acc[:, :step] = acc[:, :step] + acc[:, step:2 * step]
    return acc[:, 0].copy()


def rel_l2(y, ref) -> float:
    y = np.asarray(y, np.float64)
    ref = np.asarray(ref, np.float64)
    den = float(np.sqrt(np.sum(ref * ref)))
    num = float(np.sqrt(np.sum((y - ref) ** 2)))
    return num / den if den > 0 else num


# --------------------------------------------------------------------------------------
# seeded synthetic blocks (the distributions the benchmark configurations name)
# --------------------------------------------------------------------------------------
def _f16_bytes(v: np.ndarray) -> np.ndarray:
    return v.astype(np.float16).view(np.uint8).reshape(-1, 2)


def gen_q4k(rng: np.random.Generator, n_sb: int) -> np.ndarray:
    """d~|N(0,0.02)| f16, dmin~|N(0,0.01)| f16, 12 uniform scale bytes, 128 uniform nibble bytes."""
    blk = np.empty((n_sb, Q4K_BYTES), np.uint8)
    blk[:, 0:2] = _f16_bytes(np.abs(rng.normal(0.0, 0.02, n_sb)))
    blk[:, 2:4] = _f16_bytes(np.abs(rng.normal(0.0, 0.01, n_sb)))
    blk[:, 4:] = rng.integers(0, 256, (n_sb, Q4K_BYTES - 4), dtype=np.uint8)
    return blk.reshape(-1)


def gen_q5k(rng: np.random.Generator, n_sb: int) -> np.ndarray:
    blk = np.empty((n_sb, Q5K_BYTES), np.uint8)
    blk[:, 0:2] = _f16_bytes(np.abs(rng.normal(0.0, 0.02, n_sb)))
    blk[:, 2:4] = _f16_bytes(np.abs(rng.normal(0.0, 0.01, n_sb)))
    blk[:, 4:] = rng.integers(0, 256, (n_sb, Q5K_BYTES - 4), dtype=np.uint8)
    return blk.reshape(-1)


def gen_q6k(rng: np.random.Generator, n_sb: int) -> np.ndarray:
    """ql/qh uniform bits, 16 int8 scales uniform -32..31, d~|N(0,0.02)| f16."""
    blk = np.empty((n_sb, Q6K_BYTES), np.uint8)
    blk[:, 0:192] = rng.integers(0, 256, (n_sb, 192), dtype=np.uint8)
    blk[:, 192:208] = rng.integers(-32, 32, (n_sb, 16), dtype=np.int8).view(np.uint8)
    blk[:, 208:210] = _f16_bytes(np.abs(rng.normal(0.0, 0.02, n_sb)))
    return blk.reshape(-1)


def gen_q4k_simplified(rng: np.random.Generator, n_blocks: int) -> np.ndarray:
    """Seeded simplified blocks: scale = f16(|N(0, 0.02)|), nibbles uniform."""
    b = np.empty((n_blocks, Q4K_SIMPLE_BYTES), np.uint8)
    b[:, 0:2] = _f16_bytes(np.abs(rng.normal(0.0, 0.02, n_blocks)))
    b[:, 2:] = rng.integers(0, 256, (n_blocks, 16), dtype=np.uint8)
    return b.reshape(-1)


GEN = {"q4k": gen_q4k, "q5k": gen_q5k, "q6k": gen_q6k}


def gen_matrix(fmt: str, seed: int, n: int, k: int) -> np.ndarray:
    return GEN[fmt](np.random.default_rng(seed), n * (k // SUPER_BLOCK))


def gen_x(seed: int, *shape: int) -> np.ndarray:
    return np.random.default_rng(seed).standard_normal(shape).astype(np.float32)
