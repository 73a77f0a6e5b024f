"""GPU parity: neighbouring independent entries of a GEMV list share one launch; the results must have the
same bits as with one launch per entry (fusing switched off), and match the fp64 oracle."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import _ffi

pytestmark = pytest.mark.gpu

TOL = 1e-5


def _tune(key, value):
    assert _ffi.lib().trn_set_tuning(key.encode(), int(value)) == 0


def _run(gpu, specs, x_len, group_off, plan_out=None):
    ctx, stream = gpu
    host = {"x": kq.gen_x(1, x_len)}
    bufs = {"x": t.GpuBuffer.from_host(ctx, host["x"])}
    mats, keep, batch = [], [], t.GemvBatch()
    for i, (fmt, n, k, src, dst, flags) in enumerate(specs):
        if dst not in bufs:
            bufs[dst] = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
        m = kq.gen_matrix(fmt, 900 + i, n, k)
        mats.append(m)
        w = t.GpuBuffer.from_host(ctx, m)
        keep.append(w)            # the list holds raw pointers: the buffers must outlive the launch
        batch.add(fmt, k, n, bufs[dst], w, bufs[src], flags)
    _tune("group_off", group_off)
    try:
        if plan_out is not None:
            plan_out.extend(batch.plan())
        batch.launch(stream)
        stream.synchronize()
    finally:
        _tune("group_off", 0)
    return {k: v.copy_to_host() for k, v in bufs.items()}, mats


CASES = {
    # q, k, v share x; o depends on q; gate, up share o's output; down depends on gate
    "layer": ([("q4k", 1024, 1024, "x", "q", 1), ("q4k", 1024, 1024, "x", "k", 1), ("q4k", 1024, 1024, "x", "v", 1),
               ("q4k", 1024, 1024, "q", "o", 1), ("q4k", 2816, 1024, "o", "g", 1), ("q4k", 2816, 1024, "o", "u", 1),
               ("q6k", 1024, 2816, "g", "d", 1)], 1024),
    # mixed formats and ragged row counts in one group; five independent entries (a group holds four)
    "mixed": ([("q4k", 37, 512, "x", "a", 0), ("q5k", 513, 512, "x", "b", 1), ("q6k", 300, 512, "x", "c", 1),
               ("q4k", 64, 512, "x", "d", 0), ("q5k", 129, 512, "x", "e", 1)], 512),
    # different k, formats and row counts in one group (workgroups sized for the widest entry)
    "mixed_k": ([("q6k", 512, 2816, "x", "a", 1), ("q4k", 1024, 1024, "x", "b", 0), ("q5k", 300, 512, "x", "c", 1),
                 ("q4k", 37, 4352, "x", "d", 1), ("q6k", 40, 256, "a", "e", 1)], 4352),
    # write-after-read and read-after-write must not be fused
    "no_fuse": ([("q4k", 512, 512, "x", "a", 1), ("q4k", 256, 768, "x", "b", 1), ("q4k", 512, 512, "a", "x2", 0),
                 ("q4k", 512, 512, "x2", "a", 0)], 768),
}


def _random_list(seed, entries=28):
    """A list whose entries read buffers that earlier entries wrote (or x) and write new or existing buffers: read-after-
    write, write-after-read and write-after-write dependencies at random, three formats, ragged row counts."""
    rng = np.random.default_rng(seed)
    sizes = {"x": 256 * int(rng.integers(1, 20))}
    written, specs = ["x"], []
    for i in range(entries):
        src = written[int(rng.integers(0, len(written)))]
        k = sizes[src] // 256 * 256
        if k == 0:
            src, k = "x", sizes["x"]
        dst = f"b{i}"
        if rng.random() < 0.35:
            cands = [b for b in sizes if b != src and b != "x"]
            if cands:
                dst = cands[int(rng.integers(0, len(cands)))]
        if dst not in sizes:
            sizes[dst] = int(rng.choice([37, 256, 300, 512, 1024, 1500, 2816, 4352, 5000]))
        specs.append((("q4k", "q5k", "q6k")[int(rng.integers(0, 3))], sizes[dst], k, src, dst, int(rng.integers(0, 2))))
        if dst not in written:
            written.append(dst)
    return specs, sizes["x"]


@pytest.mark.parametrize("seed", range(100, 105))
def test_random_lists_grouped_equal_separate(gpu, seed):
    specs, x_len = _random_list(seed)
    plan = []
    sep, _ = _run(gpu, specs, x_len, 1)
    got, _ = _run(gpu, specs, x_len, 0, plan)
    assert max(plan) + 1 < len(specs)          # something was grouped
    for name in sep:
        assert np.array_equal(sep[name].view(np.uint32), got[name].view(np.uint32)), (seed, name)


@pytest.mark.parametrize("case", sorted(CASES))
def test_grouped_equals_separate(gpu, case):
    specs, x_len = CASES[case]
    sep, _ = _run(gpu, specs, x_len, 1)
    got, mats = _run(gpu, specs, x_len, 0)
    for name in sep:
        assert np.array_equal(sep[name].view(np.uint32), got[name].view(np.uint32)), (case, name)
    # the chain against fp64, entry by entry, each on the input the GPU actually used
    final = {}
    for (fmt, n, k, src, dst, flags), m in zip(specs, mats):
        final[dst] = (fmt, n, k, src, flags, m)
    for dst, (fmt, n, k, src, flags, m) in final.items():
        if case == "no_fuse" and dst in ("a", "x2"):
            continue            # overwritten or re-read later in the list
        x = got[src][:k].astype(np.float64)
        ref = kq.dequant_matrix(fmt, m, n, k).astype(np.float64) @ x
        if flags:
            ref = ref / np.sqrt(np.mean(x * x) + 1e-6)
        assert kq.rel_l2(got[dst], ref) <= TOL, (case, dst)


@pytest.mark.parametrize("group_max", (0, 16, 11, 8))
def test_nineteen_independent_entries(gpu, group_max):
    """Nineteen independent entries of mixed formats and shapes: by default all in one launch (more than sixteen: the
    launch that takes its entries from tables in device memory), with "group_max" sixteen to a launch (every position of
    the kernel-argument table of first workgroups is used) or fewer.  Same bits as one launch per entry."""
    fmts = ("q4k", "q5k", "q6k")
    specs = [(fmts[i % 3], 33 + 41 * i, 256 * (1 + (i * 5) % 7), "x", f"y{i}", i % 2) for i in range(19)]
    sep, _ = _run(gpu, specs, 256 * 7, 1)
    _tune("group_max", group_max)
    _tune("group_window", 32)
    plan = []
    try:
        got, mats = _run(gpu, specs, 256 * 7, 0, plan)
    finally:
        _tune("group_max", 0)
        _tune("group_window", 0)
    most = {0: 19, 16: 16, 11: 11, 8: 8}[group_max]
    assert len(plan) == 19 and max(np.bincount(plan)) == most and max(plan) + 1 == -(-19 // most), plan
    for name in sep:
        assert np.array_equal(sep[name].view(np.uint32), got[name].view(np.uint32)), (group_max, name)
    for (fmt, n, k, src, dst, flags), m in zip(specs, mats):
        x = got[src][:k].astype(np.float64)
        ref = kq.dequant_matrix(fmt, m, n, k).astype(np.float64) @ x
        if flags:
            ref = ref / np.sqrt(np.mean(x * x) + 1e-6)
        assert kq.rel_l2(got[dst], ref) <= TOL, (group_max, dst)


@pytest.mark.parametrize("seed", (0, 1))
def test_many_entries_in_one_launch(gpu, seed):
    """Seventy independent entries - three formats, one to four slabs of columns, ragged and large row counts, with and
    without the normalised input - go into ONE launch whose workgroups each take pieces of several entries (or a slice
    of a large one).  Same bits as one launch per entry; every entry against fp64; a second call (the cached plan) and
    a call after the list has changed give the same again."""
    rng = np.random.default_rng(seed)
    ks = (256, 1024, 4096, 4352, 8192, 11008, 14336)
    ns = (1, 37, 300, 1024, 2817, 4096, 9000)
    specs = [(("q4k", "q5k", "q6k")[int(rng.integers(3))], int(rng.choice(ns)), int(rng.choice(ks)), "x", f"y{i}", int(rng.integers(2)))
             for i in range(70)]
    sep, _ = _run(gpu, specs, 14336, 1)
    plan = []
    got, mats = _run(gpu, specs, 14336, 0, plan)
    assert max(plan) == 0, plan                     # one launch
    for name in sep:
        assert np.array_equal(sep[name].view(np.uint32), got[name].view(np.uint32)), (seed, name)
    for (fmt, n, k, src, dst, flags), m in zip(specs, mats):
        x = got[src][:k].astype(np.float64)
        ref = kq.dequant_matrix(fmt, m, n, k).astype(np.float64) @ x
        if flags:
            ref = ref / np.sqrt(np.mean(x * x) + 1e-6)
        assert kq.rel_l2(got[dst], ref) <= TOL, (seed, dst, fmt, n, k)


@pytest.mark.parametrize("item_kb,slab_weight", [(4000, 90), (1, 1)])
def test_many_entries_whatever_the_weights_of_the_cut(gpu, item_kb, slab_weight):
    """How a large launch shares out its workgroups (the cost of a piece of work, the weight of a further slab) decides
    which workgroup takes which rows and nothing else: with a piece at 4 MB (most workgroups then get too much and the last
    ones nothing) or at nothing the results are the bits of one launch per entry."""
    rng = np.random.default_rng(7)
    specs = [(("q4k", "q5k", "q6k")[int(rng.integers(3))], int(rng.choice((1, 31, 33, 640, 2817))), int(rng.choice((256, 4096, 8192, 11008))),
              "x", f"y{i}", int(rng.integers(2))) for i in range(40)]
    sep, _ = _run(gpu, specs, 11008, 1)
    try:
        _tune("many_item_kb", item_kb)
        _tune("many_slab_weight", slab_weight)
        plan = []
        got, _ = _run(gpu, specs, 11008, 0, plan)
    finally:
        _tune("many_item_kb", 0)
        _tune("many_slab_weight", 0)
    assert max(plan) == 0, plan
    for name in sep:
        assert np.array_equal(sep[name].view(np.uint32), got[name].view(np.uint32)), name


def test_many_entries_with_q6k_streamed_through_lds(gpu):
    """A large launch of one-slab matrices in workgroups of eight waves, Q6_K streamed through LDS as well (both opt-in):
    the bits of one launch per entry."""
    rng = np.random.default_rng(11)
    specs = [(("q6k", "q4k", "q6k")[i % 3], int(rng.choice((2, 31, 640, 2817))), int(rng.choice((256, 1024, 4096))),
              "x", f"y{i}", int(rng.integers(2))) for i in range(36)]
    sep, _ = _run(gpu, specs, 4096, 1)
    try:
        _tune("gemv_stream_q6k", 1)
        _tune("many_waves", 8)
        plan = []
        got, _ = _run(gpu, specs, 4096, 0, plan)
    finally:
        _tune("gemv_stream_q6k", 0)
        _tune("many_waves", 0)
    assert max(plan) == 0, plan
    for name in sep:
        assert np.array_equal(sep[name].view(np.uint32), got[name].view(np.uint32)), name


def test_many_entries_plan_is_reused_and_replaced(gpu):
    """The cut of a list and its device tables are kept per stream for as long as the same list comes again; another list
    replaces them.  Two lists issued alternately on one stream, each twice in a row: always the bits of one launch per entry."""
    ctx, stream = gpu
    lists = []
    for li in range(2):
        specs = [(("q4k", "q6k", "q5k")[(i + li) % 3], 200 + 37 * i, 256 * (1 + (i + li) % 5), "x", f"y{i}", i % 2) for i in range(24 + 6 * li)]
        x = t.GpuBuffer.from_host(ctx, kq.gen_x(3 + li, 256 * 5))
        outs, keep, batch = [], [], t.GemvBatch()
        for i, (fmt, n, k, _, _, flags) in enumerate(specs):
            w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(fmt, 3000 + 100 * li + i, n, k))
            y = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
            keep.append(w)
            outs.append(y)
            batch.add(fmt, k, n, y, w, x, flags)
        _tune("group_off", 1)
        try:
            batch.launch(stream)
            stream.synchronize()
        finally:
            _tune("group_off", 0)
        want = [y.copy_to_host() for y in outs]
        assert max(batch.plan()) == 0
        lists.append((batch, outs, want, keep, x))
    for rep in range(3):
        for batch, outs, want, _, _ in lists:
            for again in range(2):
                for y, w0 in zip(outs, want):
                    y.copy_from_host(np.full(len(w0), np.nan, np.float32))
                batch.launch(stream)
                stream.synchronize()
                for i, (y, w0) in enumerate(zip(outs, want)):
                    assert np.array_equal(y.copy_to_host().view(np.uint32), w0.view(np.uint32)), (rep, again, i)


@pytest.mark.parametrize("seed", (0, 1, 2, 3))
def test_entries_brought_forward_keep_the_lists_meaning(gpu, seed):
    """A launch may take entries from further down the list when nothing they touch is touched by an entry they
    overtake.  Random lists over a small pool of vectors (so that read-after-write, write-after-read and
    write-after-write all occur, also in place) must leave every vector with the bits of one launch per entry."""
    rng = np.random.default_rng(seed)
    dim = 512
    names = [f"v{i}" for i in range(6)]
    specs = []
    for i in range(20):
        src, dst = rng.choice(names, 2, replace=False)
        specs.append((("q4k", "q5k", "q6k")[int(rng.integers(3))], dim, dim, str(src), str(dst), 1))

    def run(group_off):
        ctx, stream = gpu
        bufs = {nm: t.GpuBuffer.from_host(ctx, kq.gen_x(50 + j, dim)) for j, nm in enumerate(names)}
        keep, batch = [], t.GemvBatch()
        for i, (fmt, n, k, src, dst, flags) in enumerate(specs):
            w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(fmt, 7000 + 100 * seed + i, n, k))
            keep.append(w)
            batch.add(fmt, k, n, bufs[dst], w, bufs[src], flags)
        _tune("group_off", group_off)
        try:
            batch.launch(stream)
            stream.synchronize()
        finally:
            _tune("group_off", 0)
        return {nm: b.copy_to_host() for nm, b in bufs.items()}

    want, got = run(1), run(0)
    for nm in names:
        assert np.all(np.isfinite(want[nm])), nm
        assert np.array_equal(want[nm].view(np.uint32), got[nm].view(np.uint32)), (seed, nm)


def test_a_list_captured_into_a_hip_graph_replays_to_the_same_bits(gpu):
    """The default way of issuing a list allocates nothing and clears nothing, so a caller may capture it into a HIP
    graph.  Every replay, with eager launches and synchronisations in between, must give the eager result."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    ctx, stream = gpu
    specs, x_len = CASES["layer"]
    bufs = {"x": t.GpuBuffer.from_host(ctx, kq.gen_x(1, x_len))}
    keep, batch = [], t.GemvBatch()
    for i, (fmt, n, k, src, dst, flags) in enumerate(specs):
        if dst not in bufs:
            bufs[dst] = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
        w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(fmt, 900 + i, n, k))
        keep.append(w)
        batch.add(fmt, k, n, bufs[dst], w, bufs[src], flags)
    batch.launch(stream)                       # eager: loads the code object, gives the expected bits
    stream.synchronize()
    want = {nm: b.copy_to_host() for nm, b in bufs.items()}
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream.raw(), 0) == 0
    batch.launch(stream)
    assert hip.hipStreamEndCapture(stream.raw(), C.byref(graph)) == 0
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    try:
        for rep in range(3):
            for nm in bufs:
                if nm != "x":
                    bufs[nm].copy_from_host(np.full(len(want[nm]), np.nan, np.float32))
            assert hip.hipGraphLaunch(gexec, stream.raw()) == 0
            stream.synchronize()
            for nm in bufs:
                assert np.array_equal(bufs[nm].copy_to_host().view(np.uint32), want[nm].view(np.uint32)), (rep, nm)
            batch.launch(stream)               # eager work between the replays
            stream.synchronize()
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)


def test_a_capture_of_a_list_issued_before_takes_its_large_launch(gpu):
    """A list of more than sixteen independent entries that the stream has issued eagerly is captured as the ONE launch it
    is (its tables exist already: nothing is allocated under capture); the replays give the eager bits, also after the
    plan has been pushed out of the stream's cache by nine other lists - the tables a graph may read are kept."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    hip.hipStreamBeginCapture.argtypes = [C.c_void_p, C.c_int]
    hip.hipStreamEndCapture.argtypes = [C.c_void_p, C.POINTER(C.c_void_p)]
    hip.hipGraphInstantiate.argtypes = [C.POINTER(C.c_void_p), C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
    hip.hipGraphLaunch.argtypes = [C.c_void_p, C.c_void_p]
    hip.hipGraphGetNodes.argtypes = [C.c_void_p, C.c_void_p, C.POINTER(C.c_size_t)]
    hip.hipGraphExecDestroy.argtypes = [C.c_void_p]
    hip.hipGraphDestroy.argtypes = [C.c_void_p]
    ctx, stream = gpu

    def make(seed, entries):
        x = t.GpuBuffer.from_host(ctx, kq.gen_x(seed, 4096))
        outs, keep, batch = [], [x], t.GemvBatch()
        for i in range(entries):
            fmt, n, k = ("q4k", "q6k", "q5k")[i % 3], 100 + 61 * i, 256 * (1 + i % 16)
            w = t.GpuBuffer.from_host(ctx, kq.gen_matrix(fmt, seed * 100 + i, n, k))
            y = t.GpuBuffer.from_host(ctx, np.full(n, np.nan, np.float32))
            keep.append(w)
            outs.append(y)
            batch.add(fmt, k, n, y, w, x, i % 2)
        return batch, outs, keep

    batch, outs, keep = make(5, 24)
    assert max(batch.plan()) == 0                      # one launch
    batch.launch(stream)                               # eager: makes the plan and its tables
    stream.synchronize()
    want = [y.copy_to_host() for y in outs]
    assert all(np.all(np.isfinite(w)) for w in want)
    graph, gexec = C.c_void_p(), C.c_void_p()
    assert hip.hipStreamBeginCapture(stream.raw(), 0) == 0
    batch.launch(stream)
    assert hip.hipStreamEndCapture(stream.raw(), C.byref(graph)) == 0
    nodes = C.c_size_t(0)
    assert hip.hipGraphGetNodes(graph, None, C.byref(nodes)) == 0 and nodes.value == 1, nodes.value
    assert hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, 0) == 0
    others = []
    try:
        for rep in range(4):
            for y, w in zip(outs, want):
                y.copy_from_host(np.full(len(w), np.nan, np.float32))
            assert hip.hipGraphLaunch(gexec, stream.raw()) == 0
            stream.synchronize()
            for i, (y, w) in enumerate(zip(outs, want)):
                assert np.array_equal(y.copy_to_host().view(np.uint32), w.view(np.uint32)), (rep, i)
            if rep == 1:                               # nine other lists: the captured list's plan leaves the cache
                for s in range(9):
                    others.append(make(20 + s, 18 + s))
                    others[-1][0].launch(stream)
                stream.synchronize()
            batch.launch(stream)                       # eager work between the replays (after rep 1: a new plan, new tables)
            stream.synchronize()
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
