"""incremental_attention (attention.rs:808-1095): single-query attention over a KV cache.  Oracle pins on the CPU, parity of
the GPU kernel through the C ABI: 1e-5 relative L2 per call against fp64, and no worse than 1.5x the f32 recurrence of the
reference evaluated position by position."""
import numpy as np
import pytest

import trueno_amd as t
from oracle import glue
from oracle import kquant as kq

TOL = 1e-5


def _case(seed, heads, kv_heads, max_seq, dim, spread=1.0):
    rng = np.random.default_rng(seed)
    q = (rng.standard_normal((heads, dim)) * spread).astype(np.float32)
    k = rng.standard_normal((kv_heads, max_seq, dim)).astype(np.float32)
    v = rng.standard_normal((kv_heads, max_seq, dim)).astype(np.float32)
    return q, k, v


def test_names_and_fields_follow_the_reference():
    a = t.IncrementalAttentionKernel(2048, 64, 32)
    assert a.name() == "incremental_attention" and not a.is_gqa() and a.num_kv_heads == 32      # attention.rs:823-831, 862
    assert abs(a.scale - 0.125) < 1e-7                                                          # 1/sqrt(head_dim), :849
    g = t.IncrementalAttentionKernel.with_gqa(2048, 128, 32, 8)
    assert g.is_gqa() and g.num_kv_heads == 8
    assert g.launch_config().grid == (32, 1, 1) and g.launch_config().block == (32, 1, 1)


def test_oracle_special_cases():
    q, k, v = _case(1, 4, 2, 16, 8)
    assert np.allclose(glue.attention_fp64(q, k, v, 1), v[[0, 0, 1, 1], 0])          # one position: its value; GQA map 0,0,1,1
    k_same = np.repeat(k[:, :1], 16, axis=1)
    assert np.allclose(glue.attention_fp64(q, k_same, v, 16), v[[0, 0, 1, 1]].mean(axis=1))      # equal keys: the mean
    k_peak = k.copy()
    k_peak[:, 5] = 0.0
    q_big = np.zeros_like(q)
    q_big[:, 0] = 1000.0
    k_peak[:, :, 0] = -1.0
    k_peak[:, 5, 0] = 1.0                                                             # position 5 wins by e^(2000*scale)
    assert np.allclose(glue.attention_fp64(q_big, k_peak, v, 16), v[[0, 0, 1, 1], 5])
    got = glue.attention_ref_order(q, k, v, 16)
    assert kq.rel_l2(got, glue.attention_fp64(q, k, v, 16)) <= 5e-7
    # positions beyond seq_len do not matter
    k2, v2 = k.copy(), v.copy()
    k2[:, 9:], v2[:, 9:] = 7.0, -3.0
    assert np.array_equal(glue.attention_fp64(q, k, v, 9), glue.attention_fp64(q, k2, v2, 9))


@pytest.mark.gpu
@pytest.mark.parametrize("heads,kv_heads,max_seq,seq,dim", [(32, 32, 256, 256, 64), (32, 8, 512, 300, 128), (4, 1, 64, 1, 32),
                                                             (8, 4, 4096, 4096, 128), (3, 3, 100, 37, 20), (2, 2, 2100, 2049, 256),
                                                             (16, 16, 128, 100, 4)])
def test_gpu_incremental_attention(gpu, heads, kv_heads, max_seq, seq, dim):
    ctx, stream = gpu
    q, k, v = _case(heads * 1000 + seq, heads, kv_heads, max_seq, dim, spread=2.0)
    dq, dk, dv = (t.GpuBuffer.from_host(ctx, a.reshape(-1)) for a in (q, k, v))
    do = t.GpuBuffer.from_host(ctx, np.full(heads * dim, np.nan, np.float32))
    kern = t.IncrementalAttentionKernel.with_gqa(max_seq, dim, heads, kv_heads)
    kern.launch(stream, dq, dk, dv, do, seq)
    stream.synchronize()
    got = do.copy_to_host().reshape(heads, dim)
    want = glue.attention_fp64(q, k, v, seq)
    err = kq.rel_l2(got, want)
    assert err <= TOL, err
    if seq <= 300 and heads * dim >= 256:
        ref = kq.rel_l2(glue.attention_ref_order(q, k, v, seq), want)
        assert err <= 1.5 * ref + 1e-9, (err, ref)
    again = t.GpuBuffer.from_host(ctx, np.zeros(heads * dim, np.float32))
    kern.launch(stream, dq, dk, dv, again, seq)                     # the chunks are merged in chunk order: same bits
    stream.synchronize()
    assert np.array_equal(again.copy_to_host().view(np.uint32), got.reshape(-1).view(np.uint32))


@pytest.mark.gpu
def test_gpu_attention_by_name_extremes_and_bad_arguments(gpu):
    ctx, stream = gpu
    module = t.CudaModule.from_builtin(ctx)
    heads, dim, max_seq, seq = 8, 64, 128, 128
    q, k, v = _case(5, heads, heads, max_seq, dim)
    q *= 30.0                                                       # scores of a few hundred: the running maximum matters
    dq, dk, dv = (t.GpuBuffer.from_host(ctx, a.reshape(-1)) for a in (q, k, v))
    do = t.GpuBuffer.from_host(ctx, np.zeros(heads * dim, np.float32))
    kern = t.IncrementalAttentionKernel(max_seq, dim, heads)
    kern.launch_by_name(stream, module, dq, dk, dv, do, seq)
    stream.synchronize()
    got = do.copy_to_host().reshape(heads, dim)
    assert np.all(np.isfinite(got)) and kq.rel_l2(got, glue.attention_fp64(q, k, v, seq)) <= TOL
    L = t._ffi.lib()
    args = (dq.as_ptr(), dk.as_ptr(), dv.as_ptr(), do.as_ptr())
    assert L.trn_incremental_attention(stream.raw(), *args, 0, dim, heads, heads, max_seq, 0.125) != 0          # no position
    assert L.trn_incremental_attention(stream.raw(), *args, max_seq + 1, dim, heads, heads, max_seq, 0.125) != 0
    assert L.trn_incremental_attention(stream.raw(), *args, seq, 66, heads, heads, max_seq, 0.125) != 0        # head_dim % 4
    assert L.trn_incremental_attention(stream.raw(), *args, seq, 512, heads, heads, max_seq, 0.125) != 0
    assert L.trn_incremental_attention(stream.raw(), *args, seq, dim, heads, heads + 1, max_seq, 0.125) != 0
    assert L.trn_incremental_attention(stream.raw(), 0, dk.as_ptr(), dv.as_ptr(), do.as_ptr(), seq, dim, heads, heads, max_seq, 0.125) != 0
