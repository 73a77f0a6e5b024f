"""Writes tests/golden/kquant_golden.npz: a few super-blocks per format and the f32 bit patterns
both decode families must produce for them.

The reference holds no numeric vector for this path (its tests only inspect PTX text), so these
vectors come from the numpy oracle (oracle/kquant.py) and are accepted only if the independently
written C oracle (oracle/kquant_ref.c) produces the same bits.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import kquant as kq  # noqa: E402
from oracle.cref import COracle  # noqa: E402


def main() -> None:
    co = COracle()
    rng = np.random.default_rng(20240607)
    out = {}
    for fmt in ("q4k", "q5k", "q6k"):
        sb = kq.SB_BYTES[fmt]
        blk = kq.GEN[fmt](rng, 12).reshape(12, sb).copy()
        d_offs = (208,) if fmt == "q6k" else (0, 2)
        # forced f16 fields: zero, smallest subnormal, largest subnormal, smallest normal, 1.0, max
        for i, bits in enumerate((0x0000, 0x0001, 0x03FF, 0x0400, 0x3C00, 0x7BFF)):
            for o in d_offs:
                blk[i, o:o + 2] = np.array([bits], np.uint16).view(np.uint8)
        blk[6, :] = 0
        blk[7, :] = 0xFF
        if fmt == "q6k":
            blk[7, 208:210] = np.array([0x3C00], np.uint16).view(np.uint8)  # 0xFFFF is a NaN
        else:
            blk[7, 0:4] = np.array([0x3C00, 0x3800], np.uint16).view(np.uint8)
        out[f"{fmt}_blocks"] = blk.reshape(-1)
        for policy in (0, 1):
            w = kq.DEQUANT[(fmt, policy)](blk.reshape(-1))
            wc = co.dequant(fmt, blk.reshape(-1), policy)
            assert np.array_equal(w.view(np.uint32), wc.view(np.uint32)), (fmt, policy)
            out[f"{fmt}_w{policy}_bits"] = w.view(np.uint32).reshape(-1)
    # one tiny GEMV per format: W (3 x 512), x, fp64 product
    for fmt in ("q4k", "q5k", "q6k"):
        buf = kq.gen_matrix(fmt, 99, 3, 512)
        x = kq.gen_x(98, 512)
        out[f"{fmt}_gemv_w"] = buf
        out[f"{fmt}_gemv_x"] = x
        out[f"{fmt}_gemv_y64"] = kq.gemv_fp64(kq.dequant_matrix(fmt, buf, 3, 512), x)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "kquant_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
