"""GPU parity of the three ways a list is issued (grouped launches, one launch per entry, resident phases): the
same bits for every format, ragged row counts and K > 4096 (several waves per row)."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import _ffi

pytestmark = pytest.mark.gpu


def _tune(key, value):
    assert _ffi.lib().trn_set_tuning(key.encode(), int(value)) == 0


def _run(gpu, specs, x_len, mode):
    """specs: list of (fmt, n, k, src, dst, flags); buffers by name, 'x' is the input"""
    ctx, stream = gpu
    bufs = {"x": t.GpuBuffer.from_host(ctx, kq.gen_x(1, x_len))}
    ws, batch = [], t.GemvBatch()
    for i, (fmt, n, k, src, dst, flags) in enumerate(specs):
        if dst not in bufs:
            bufs[dst] = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
        w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(fmt, 500 + i, n, k))
        ws.append(w)
        batch.add(fmt, k, n, bufs[dst], w, bufs[src], flags)
    for key, val in mode.items():
        _tune(key, val)
    try:
        batch.launch(stream)
        stream.synchronize()
        batch.launch(stream)          # a second launch of the same list
        stream.synchronize()
    finally:
        for key in mode:
            _tune(key, 0)
    return {k: v.copy_to_host() for k, v in bufs.items()}


CASES = {
    "q4k_chain": ([("q4k", 4096, 4096, "x", "a", 1), ("q4k", 4096, 4096, "x", "b", 1), ("q4k", 4096, 4096, "a", "c", 1),
                   ("q4k", 11008, 4096, "c", "d", 1), ("q4k", 11008, 4096, "c", "e", 0)], 4096),
    "q6k_big_k": ([("q4k", 11008, 4096, "x", "g", 1), ("q6k", 4096, 11008, "g", "d", 1), ("q6k", 32000, 4096, "d", "l", 1)], 4096),
    "q5k_mixed": ([("q5k", 1000, 1024, "x", "a", 1), ("q5k", 1024, 1024, "x", "b", 0), ("q6k", 1024, 1024, "x", "c", 1),
                   ("q4k", 512, 1024, "c", "d", 1), ("q5k", 4096, 11008, "g0", "e", 0)], 1024),
    "ragged": ([("q4k", 37, 512, "x", "a", 0), ("q4k", 513, 512, "x", "b", 1), ("q5k", 300, 512, "b", "c", 1),
                ("q6k", 264, 768, "d0", "e", 1)], 768),
}


@pytest.mark.parametrize("case", sorted(CASES))
def test_issue_modes_give_the_same_bits(gpu, case):
    specs, x_len = CASES[case]
    ctx, _ = gpu
    # inputs named g0/d0 are extra seeded vectors
    specs2 = []
    for fmt, n, k, src, dst, flags in specs:
        specs2.append((fmt, n, k, "x" if src in ("g0", "d0") and k <= x_len else src, dst, flags))
    if case == "q5k_mixed":
        specs2[-1] = ("q5k", 4096, 1024, "x", "e", 0)
    ref = _run(gpu, specs2, x_len, {"batch_mode": 0})
    got = _run(gpu, specs2, x_len, {"group_off": 1})
    for name in ref:
        assert np.array_equal(ref[name].view(np.uint32), got[name].view(np.uint32)), (case, name, "one launch per entry")
    old = _run(gpu, specs2, x_len, {"batch_mode": 1})
    for name in ref:
        assert np.array_equal(ref[name].view(np.uint32), old[name].view(np.uint32)), (case, name, "resident phases")
