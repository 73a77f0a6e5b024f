"""GGUF adapter: the GGML Q5_K block against an independent scalar restatement of the public format, the re-pack into the
reference's Q5_K layout (oracle and GPU kernel, bit for bit), and a synthetic GGUF file read back, uploaded and multiplied.

No GGUF file and no ggml/gguf package exist in this environment; the file is written here from the published format
(header, key/value metadata, tensor infos, aligned data section) and the blocks are random bytes with sane f16 headers."""
import struct

import numpy as np
import pytest

import trueno_amd as t
from oracle import kquant as kq
from trueno_amd import gguf

TOL = 1e-5


def _ggml_q5k_blocks(seed, n_sb):
    rng = np.random.default_rng(seed)
    blk = rng.integers(0, 256, (n_sb, 176), dtype=np.uint8)
    blk[:, 0:2] = np.abs(rng.normal(0, 0.02, n_sb)).astype(np.float16).view(np.uint8).reshape(n_sb, 2)
    blk[:, 2:4] = np.abs(rng.normal(0, 0.01, n_sb)).astype(np.float16).view(np.uint8).reshape(n_sb, 2)
    return blk.reshape(-1)


def _dequantize_row_q5_K_scalar(block: bytes):
    """ggml's dequantize_row_q5_K for one block, written from the public definition with its loop structure (64 values
    per step, two masks walking up the bits of qh), independent of the vectorised oracle."""
    d = float(np.frombuffer(block[0:2], np.float16)[0])
    dmin = float(np.frombuffer(block[2:4], np.float16)[0])
    scales, qh, ql = block[4:16], block[16:48], block[48:176]

    def scale_min(j):
        if j < 4:
            return scales[j] & 63, scales[j + 4] & 63
        return (scales[j + 4] & 0xF) | ((scales[j - 4] >> 6) << 4), (scales[j + 4] >> 4) | ((scales[j] >> 6) << 4)

    out, is_, u1, u2, qo = [], 0, 1, 2, 0
    for _ in range(0, 256, 64):
        sc, m = scale_min(is_)
        d1, m1 = np.float32(d) * np.float32(sc), np.float32(dmin) * np.float32(m)
        sc, m = scale_min(is_ + 1)
        d2, m2 = np.float32(d) * np.float32(sc), np.float32(dmin) * np.float32(m)
        for l in range(32):
            out.append(d1 * np.float32((ql[qo + l] & 0xF) + (16 if qh[l] & u1 else 0)) - m1)
        for l in range(32):
            out.append(d2 * np.float32((ql[qo + l] >> 4) + (16 if qh[l] & u2 else 0)) - m2)
        qo, is_, u1, u2 = qo + 32, is_ + 2, u1 << 2, u2 << 2
    return np.array(out, np.float32)


def test_ggml_q5k_oracle_against_the_scalar_restatement():
    blocks = _ggml_q5k_blocks(1, 6)
    got = kq.dequant_q5k_ggml(blocks)
    for i in range(6):
        want = _dequantize_row_q5_K_scalar(bytes(blocks[176 * i:176 * (i + 1)]))
        assert np.array_equal(got[i].view(np.uint32), want.view(np.uint32))


def test_repack_keeps_every_value():
    blocks = _ggml_q5k_blocks(2, 40)
    ref_layout = kq.q5k_ggml_to_reference(blocks)
    assert np.array_equal(kq.dequant_q5k(ref_layout).view(np.uint32), kq.dequant_q5k_ggml(blocks).view(np.uint32))
    # one-hot: a single fifth bit of GGML's qh[l], bit j, lands on value 32 j + l
    one = np.zeros(176, np.uint8)
    one[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    one[4] = 1                                              # scale of sub-block 0 = 1; all other scales 0
    one[16 + 9] = 1 << 0                                    # fifth bit of value 9 (sub-block 0)
    w = kq.dequant_q5k(kq.q5k_ggml_to_reference(one))[0]
    assert w[9] == 16.0 and np.count_nonzero(w) == 1


# ---- a synthetic GGUF file ---------------------------------------------------------------------

def _gguf_string(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, tensors, alignment=64):
    """tensors: list of (name, dims (ne0 first), ggml type, bytes)."""
    kv = [("general.architecture", 8, "llama"), ("general.alignment", 4, alignment), ("test.floats", 9, (6, [1.5, 2.5]))]
    out = struct.pack("<IIQQ", gguf.GGUF_MAGIC, 3, len(tensors), len(kv))
    for key, vt, val in kv:
        out += _gguf_string(key) + struct.pack("<I", vt)
        if vt == 8:
            out += _gguf_string(val)
        elif vt == 4:
            out += struct.pack("<I", val)
        else:
            et, items = val
            out += struct.pack("<IQ", et, len(items)) + b"".join(struct.pack("<f", v) for v in items)
    offsets, pos = [], 0
    for _, _, _, data in tensors:
        offsets.append(pos)
        pos = (pos + len(data) + alignment - 1) // alignment * alignment
    for (name, dims, gtype, _), off in zip(tensors, offsets):
        out += _gguf_string(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", gtype, off)
    out += b"\0" * ((len(out) + alignment - 1) // alignment * alignment - len(out))
    body = bytearray(pos)
    for (_, _, _, data), off in zip(tensors, offsets):
        body[off:off + len(data)] = data
    with open(path, "wb") as f:
        f.write(out + bytes(body))


def _make_file(tmp_path):
    n, k = 96, 512
    q4 = kq.gen_matrix("q4k", 11, n, k)
    q6 = kq.gen_matrix("q6k", 12, n, k)
    q5 = _ggml_q5k_blocks(13, n * k // 256)
    norm = kq.gen_x(14, k)
    path = str(tmp_path / "synthetic.gguf")
    write_gguf(path, [("blk.0.attn_q.weight", (k, n), gguf.GGML_Q4_K, q4.tobytes()),
                      ("blk.0.attn_norm.weight", (k,), gguf.GGML_F32, norm.tobytes()),
                      ("blk.0.ffn_up.weight", (k, n), gguf.GGML_Q5_K, q5.tobytes()),
                      ("output.weight", (k, n), gguf.GGML_Q6_K, q6.tobytes()),
                      ("other.f16", (8,), gguf.GGML_F16, np.zeros(8, np.float16).tobytes())])
    return path, n, k, q4, q5, q6, norm


def test_reader_finds_tensors_and_metadata(tmp_path):
    path, n, k, q4, q5, q6, norm = _make_file(tmp_path)
    with gguf.GgufFile(path) as f:
        assert f.version == 3 and f.metadata["general.architecture"] == "llama" and f.metadata["test.floats"] == [1.5, 2.5]
        info = f.tensors["blk.0.attn_q.weight"]
        assert (info.fmt, info.k, info.n, info.nbytes) == ("q4k", k, n, n * (k // 256) * 144)
        assert f.tensors["output.weight"].fmt == "q6k" and f.tensors["blk.0.ffn_up.weight"].fmt == "q5k"
        assert np.array_equal(f.tensor_bytes("blk.0.attn_q.weight"), q4)
        assert np.array_equal(f.tensor_bytes("output.weight"), q6)
        assert np.array_equal(f.tensor_bytes("blk.0.attn_norm.weight").view(np.float32), norm)
        assert all(t_.offset % 64 == 0 for t_ in f.tensors.values())
    with open(path, "r+b") as fh:                       # a truncated file is refused, not read past its end
        fh.truncate(1000)
    with pytest.raises(t.GpuError):
        gguf.GgufFile(path)
    bad = tmp_path / "bad.gguf"
    bad.write_bytes(b"GGML" + b"\0" * 64)
    with pytest.raises(t.GpuError):
        gguf.GgufFile(str(bad))


@pytest.mark.gpu
def test_gpu_repack_is_bit_exact_also_in_place(gpu):
    ctx, stream = gpu
    blocks = _ggml_q5k_blocks(21, 1000)
    src = t.GpuBuffer.from_host(ctx, blocks)
    dst = t.GpuBuffer.from_host(ctx, np.zeros_like(blocks))
    L = t._ffi.lib()
    assert L.trn_q5k_from_ggml(stream.raw(), dst.as_ptr(), src.as_ptr(), 1000) == 0
    assert L.trn_q5k_from_ggml(stream.raw(), src.as_ptr(), src.as_ptr(), 1000) == 0
    stream.synchronize()
    want = kq.q5k_ggml_to_reference(blocks)
    assert np.array_equal(dst.copy_to_host(), want)
    assert np.array_equal(src.copy_to_host(), want)
    assert L.trn_q5k_from_ggml(stream.raw(), 0, 0, 0) == 0 and L.trn_q5k_from_ggml(stream.raw(), 0, src.as_ptr(), 1) != 0


@pytest.mark.gpu
def test_gpu_gemv_on_tensors_from_a_gguf_file(gpu, tmp_path):
    ctx, stream = gpu
    path, n, k, q4, q5, q6, norm = _make_file(tmp_path)
    x = kq.gen_x(30, k)
    dx = t.GpuBuffer.from_host(ctx, x)
    with gguf.GgufFile(path) as f:
        for name, K, w64 in (("blk.0.attn_q.weight", t.Q4KGemvKernel, kq.dequant_matrix("q4k", q4, n, k)),
                             ("blk.0.ffn_up.weight", t.Q5KGemvKernel, kq.dequant_q5k_ggml(q5).reshape(n, k)),
                             ("output.weight", t.Q6KGemvKernel, kq.dequant_matrix("q6k", q6, n, k))):
            info = f.tensors[name]
            w = f.upload(ctx, stream, name)
            y = t.GpuBuffer.from_host(ctx, np.zeros(info.n, np.float32))
            K(info.k, info.n).launch(stream, y, w, dx)
            stream.synchronize()
            assert kq.rel_l2(y.copy_to_host(), w64.astype(np.float64) @ x.astype(np.float64)) <= TOL, name
        g = f.upload(ctx, stream, "blk.0.attn_norm.weight")
        assert np.array_equal(g.copy_to_host(), norm)
        with pytest.raises(t.GpuError):
            f.upload(ctx, stream, "other.f16")
