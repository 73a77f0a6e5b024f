"""GPU parity of the benchmark's own list (trueno_amd.decode_pass, the list bench.py times): three layers and the head
at the 7B shapes with the activation buffers shared by all layers, in the library's default mode (grouped launches,
entries brought forward across layers).  Bit for bit against one launch per entry and against the resident executor;
the last layer's outputs and the logits within 1e-5 relative L2 of fp64 on their ACTUAL inputs."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import _ffi
from trueno_amd.decode_pass import HEAD, LAYER_MATS, DecodePass

pytestmark = pytest.mark.gpu
TOL = 1e-5
LAYERS = 3


def _tune(key, value):
    assert _ffi.lib().trn_set_tuning(key.encode(), int(value)) == 0


@pytest.fixture(scope="module")
def decode_pass(gpu):
    ctx, _ = gpu
    host_last, weights = {}, []
    for layer in range(LAYERS):
        mats = {}
        for mi, (name, fmt, n, k) in enumerate(LAYER_MATS):
            host = kq.gen_matrix(fmt, 1234 + 100 * layer + mi, n, k)
            mats[name] = t.GpuBuffer.from_host(ctx, host)
            if layer == LAYERS - 1:
                host_last[name] = host
        weights.append(mats)
    host_head = kq.gen_matrix(HEAD[1], 999, HEAD[2], HEAD[3])
    xs_host = [kq.gen_x(4321 + layer, 4096) for layer in range(LAYERS)]
    p = DecodePass(ctx, weights, t.GpuBuffer.from_host(ctx, host_head), [t.GpuBuffer.from_host(ctx, x) for x in xs_host])
    return p, host_last, host_head, xs_host


def _snapshot(p):
    out = {nm: b.copy_to_host() for nm, b in p.act.items()}
    out["logits"] = p.logits.copy_to_host()
    return out


def _norm64(v, eps=1e-6):
    v = v.astype(np.float64)
    return v / np.sqrt(np.mean(v * v) + eps)


@pytest.mark.parametrize("flow", ("fresh_x", "strict"))
def test_bench_list_default_mode(gpu, decode_pass, flow):
    ctx, stream = gpu
    p, host_last, host_head, xs_host = decode_pass
    batch = p.build(flow)
    plan = batch.plan()
    assert len(plan) == 7 * LAYERS + 1 and max(plan) + 1 < len(plan), "the default mode must share launches"
    print(f"{flow}: {len(plan)} entries in {max(plan) + 1} launches", flush=True)
    batch.launch(stream)
    stream.synchronize()
    got = _snapshot(p)
    for key, label in (("group_off", "one launch per entry"), ("batch_mode", "resident executor")):
        _tune(key, 1)
        try:
            batch.launch(stream)
            stream.synchronize()
        finally:
            _tune(key, 0)
        other = _snapshot(p)
        for nm in got:
            assert np.array_equal(got[nm].view(np.uint32), other[nm].view(np.uint32)), (flow, nm, label)
    # fp64 on the actual inputs: what the GPU itself produced one step earlier
    w = {nm: kq.dequant_matrix(fmt, host_last[nm], n, k) for nm, fmt, n, k in LAYER_MATS}
    if flow == "fresh_x":
        x = xs_host[LAYERS - 1].astype(np.float64)
        want = {"q": w["q"] @ x, "k": w["k"] @ x, "v": w["v"] @ x, "gate": w["gate"] @ x, "up": w["up"] @ x,
                "o": w["o"] @ _norm64(got["q"]), "down": w["down"] @ _norm64(got["gate"])}
    else:
        want = {"o": w["o"] @ _norm64(got["q"]), "gate": w["gate"] @ _norm64(got["o"]), "up": w["up"] @ _norm64(got["o"]),
                "down": w["down"] @ _norm64(got["gate"])}
    del w
    want["logits"] = kq.dequant_matrix(HEAD[1], host_head, HEAD[2], HEAD[3]) @ _norm64(got["down"])
    for nm, ref in want.items():
        err = kq.rel_l2(got[nm], ref)
        print(f"  {flow} {nm}: rel-L2 {err:.2e}", flush=True)
        assert err <= TOL, (flow, nm, err)


def test_buffers_per_layer_give_the_same_bits_in_fewer_launches(gpu, decode_pass):
    """The same data flow with activation buffers of its own for every layer: the library brings independent entries
    of neighbouring layers together, and every layer's outputs and the logits are those of the shared-buffer pass
    (whose last layer is still in its buffers), bit for bit."""
    ctx, stream = gpu
    p = decode_pass[0]
    shared = p.build("fresh_x")
    shared.launch(stream)
    stream.synchronize()
    want = _snapshot(p)
    own = p.build("fresh_x_own_buffers")
    assert max(own.plan()) < max(shared.plan()), (own.plan(), shared.plan())
    p.logits.copy_from_host(np.zeros(HEAD[2], np.float32))
    own.launch(stream)
    stream.synchronize()
    assert np.array_equal(p.logits.copy_to_host().view(np.uint32), want["logits"].view(np.uint32))
    for nm, b in p.act_of_layer[LAYERS - 1].items():
        assert np.array_equal(b.copy_to_host().view(np.uint32), want[nm].view(np.uint32)), nm
