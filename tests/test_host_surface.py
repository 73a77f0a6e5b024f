"""Host-side mirror of the trueno-gpu surface and the C ABI, without a GPU: names, constants,
argument order, host-side error checks, and that the library exports what the header declares."""
import ctypes
import os
import re
import subprocess

import numpy as np
import pytest

import trueno_amd as t
from trueno_amd import _ffi, kernels as K

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_kernel_names_and_constants():
    # quantize.rs tests :1972-1976, :2190-2193, :2345-2348, :2447-2450, :2750-2753, :2820-2823, :2840-2843
    assert t.QuantizeKernel(1, 2, 256).name() == "q4k_gemm_fused"
    assert t.QuantizeKernel.ggml(1, 2, 256).name() == "q4k_gemm_ggml"
    assert t.Q5KKernel(1, 2, 256).name() == "q5k_gemm_ggml"
    assert t.Q6KKernel(1, 2, 256).name() == "q6k_gemm_ggml"
    assert t.Q4KGemvKernel(256, 2).name() == "q4k_gemv_warp_reduce"
    assert t.Q5KGemvKernel(256, 2).name() == "q5k_gemv_warp_reduce"
    assert t.Q6KGemvKernel(256, 2).name() == "q6k_gemv_warp_reduce"
    assert (K.Q4K_BLOCK_SIZE, K.Q4K_SUPER_BLOCK_SIZE, K.Q4K_SUPER_BLOCK_BYTES, K.Q4K_BLOCK_BYTES) == (32, 256, 144, 18)
    assert (K.Q5K_SUPER_BLOCK_BYTES, K.Q6K_SUPER_BLOCK_BYTES) == (176, 210)


def test_constructor_argument_order_and_derived_sizes():
    g = t.Q4KGemvKernel(4096, 11008)          # (k, n): quantize.rs:1171
    assert (g.k, g.n) == (4096, 11008) and g.num_super_blocks_per_row() == 16   # :2756-2761
    assert g.weight_bytes() == 11008 * 16 * 144
    q = t.QuantizeKernel.ggml(4, 14336, 4096)  # (m, n, k): quantize.rs:102
    assert (q.m, q.n, q.k, q.tile_size, q.block_size) == (4, 14336, 4096, 32, 256)
    assert q.format is t.Q4KFormat.GgmlSuperBlock and q.num_super_blocks_per_row() == 16
    s = t.QuantizeKernel(4, 8, 64)
    assert s.format is t.Q4KFormat.Simplified and s.block_size == 32 and s.num_blocks_per_row() == 2
    assert t.QuantizeKernel(1, 1, 256).with_tile_size(16).tile_size == 16


def test_reference_launch_geometry_is_reported():
    cfg = t.Q6KGemvKernel(4096, 32000).launch_config()       # quantize.rs:1151-1155
    assert cfg.grid == (32000, 1, 1) and cfg.block == (32, 1, 1) and cfg.shared_mem == 0
    cfg = t.QuantizeKernel.ggml(40, 100, 256).launch_config()
    assert cfg.grid == (4, 2, 1) and cfg.block == (1024, 1, 1)
    args = t.Q4KGemvKernel(512, 7).kernel_args(0x100, 0x200, 0x300)   # (y, w, x, k_dim, n_dim) :1190-1194
    assert [a.value for a in args] == [0x100, 0x200, 0x300, 512, 7]
    assert [type(a) for a in args] == [ctypes.c_uint64] * 3 + [ctypes.c_uint32] * 2
    args = t.Q5KKernel(3, 7, 512).kernel_args(1, 2, 3)                # (a, b_quant, c, m, n, k) :644-650
    assert [a.value for a in args] == [1, 2, 3, 3, 7, 512]


def test_launch_config_helpers():
    # driver/types.rs:95-134
    c = t.LaunchConfig.linear(1000, 256)
    assert c.grid == (4, 1, 1) and c.block == (256, 1, 1) and c.shared_mem == 0
    c = t.LaunchConfig.grid_2d(3, 5, 16, 8).with_shared_mem(4096)
    assert c.grid == (3, 5, 1) and c.block == (16, 8, 1) and c.shared_mem == 4096
    assert c.total_threads() == 3 * 5 * 16 * 8
    d = t.LaunchConfig()
    assert d.grid == (1, 1, 1) and d.block == (256, 1, 1)


def test_host_side_transfer_checks_need_no_driver():
    """length mismatch and out-of-bounds partial copies are Transfer errors raised before any driver call
    (driver/memory.rs:221-227, :388-396); zero-length buffers never touch the driver (:101-107)"""
    buf = t.GpuBuffer.from_raw_parts(0x1000, 8, np.float32)     # non-owning view, never dereferenced
    with pytest.raises(t.GpuError) as e:
        buf.copy_from_host(np.zeros(7, np.float32))
    assert e.value.kind == "Transfer" and "Length mismatch: host 7 vs device 8" in str(e.value)
    with pytest.raises(t.GpuError) as e:
        buf.copy_from_host_at(np.zeros(4, np.float32), 5)
    assert e.value.kind == "Transfer" and "Partial copy out of bounds: offset 5 + len 4 > buffer 8" in str(e.value)
    with pytest.raises(t.GpuError):
        buf.copy_to_host_at(np.zeros(9, np.float32), 0)
    empty = t.GpuBuffer(None, 0, np.float32)
    assert empty.as_ptr() == 0 and empty.is_empty() and empty.size_bytes() == 0
    empty.copy_from_host(np.zeros(0, np.float32))
    assert empty.copy_to_host().size == 0
    meta = buf.clone_metadata()
    assert isinstance(meta, t.GpuBufferView) and meta.as_ptr() == 0x1000 and meta.len() == 8 and meta.size_bytes() == 32 and not meta.is_empty()
    other = t.GpuBuffer.from_raw_parts(0x2000, 4, np.float32)
    with pytest.raises(t.GpuError) as e:                       # memory.rs:583-594: bounds are checked before any driver call
        buf.copy_from_buffer_at_async_raw(other, 6, 0, 3, None)
    assert e.value.kind == "Transfer" and "dst out of bounds: 6 + 3 > 8" in str(e.value)
    with pytest.raises(t.GpuError) as e:
        buf.copy_from_buffer_at_async_raw(other, 0, 2, 3, None)
    assert e.value.kind == "Transfer" and "src out of bounds: 2 + 3 > 4" in str(e.value)
    buf.copy_from_buffer_at_async_raw(other, 0, 0, 0, None)    # nothing to copy: no driver call
    assert buf.as_kernel_arg().value == 0x1000
    with pytest.raises(t.GpuError) as e:
        t.QuantizeKernel(1, 1, 32).launch(None, 0, 0, 0)
    assert e.value.kind == "KernelLaunch"


def test_header_symbols_are_exported_and_bound():
    header = open(os.path.join(ROOT, "include", "trueno_hip.h")).read()
    declared = set(re.findall(r"TRN_API\s+[\w\s\*]+?\b(trn_\w+)\s*\(", header))
    assert len(declared) >= 45
    lib_path = _ffi.LIB_PATH
    assert os.path.exists(lib_path), "build the library first (make -C trueno_amd/csrc)"
    out = subprocess.run(["nm", "-D", "--defined-only", lib_path], check=True, capture_output=True, text=True).stdout
    exported = {line.split()[-1] for line in out.splitlines() if " T " in line}
    assert declared <= exported, declared - exported
    assert {s for s in exported if s.startswith("trn_")} == declared    # nothing undeclared leaks out
    assert set(_ffi.SIGNATURES) == declared
    L = _ffi.lib()
    for name in declared:
        assert getattr(L, name) is not None


def test_builtin_code_object_is_embedded_and_names_the_reference_kernels():
    L = _ffi.lib()
    img, size = ctypes.c_void_p(), ctypes.c_size_t()
    assert L.trn_builtin_image(ctypes.byref(img), ctypes.byref(size)) == 0
    blob = ctypes.string_at(img.value, size.value)
    assert blob[:4] == b"\x7fELF" and size.value > 10000
    for name in (b"q4k_gemv_warp_reduce", b"q5k_gemv_warp_reduce", b"q6k_gemv_warp_reduce",
                 b"q4k_gemm_ggml", b"q5k_gemm_ggml", b"q6k_gemm_ggml"):
        assert name in blob


def test_no_device_error_convention():
    """without a GPU every device entry returns hipErrorNoDevice (100) -> CudaNotAvailable
    (driver/sys.rs:373-391, context.rs:273-305).  On a GPU box this test checks the success path instead."""
    L = _ffi.lib()
    rc = L.trn_init(0)
    if rc == 0:
        assert t.cuda_available() and t.device_count() >= 1
        with pytest.raises(t.GpuError) as e:
            t.CudaContext(10_000)
        assert e.value.kind == "DeviceNotFound"
        return
    assert rc == 100 and L.trn_error_name(rc) == b"hipErrorNoDevice"
    assert not t.cuda_available()
    with pytest.raises(t.GpuError) as e:
        t.CudaContext(0)
    assert e.value.kind == "CudaNotAvailable"
    # argument validation happens before the device is touched
    assert L.trn_q4k_gemv(None, 1, 1, 1, 100, 4) == 1            # k % 256 != 0 -> invalid value
    assert L.trn_q4k_gemv(None, 1, 1, 1, 256, 0) == 0            # n == 0 -> no-op
    assert L.trn_q4k_dequant_f32(None, 1, 1, 1, 2) == 1          # bad policy
    assert L.trn_q4k_gemv(None, 16, 16, 16, 256, 4) == 100       # would launch: no device
    assert L.trn_mem_free(0) == 0
    assert L.trn_set_tuning(b"no_such_key", 1) == 1


def test_argument_checks_that_need_no_device():
    L = _ffi.lib()
    assert L.trn_function_set_rmsnorm(None, 4096, 1e-5) == 1           # no function handle
    assert L.trn_function_set_attention(None, 128, 32, 32, 2048, 0.1) == 1
    assert L.trn_set_tuning(b"batch_mode", 2) == 1                      # 0 = grouped launches, 1 = resident phases, nothing else
    assert L.trn_set_tuning(b"batch_mode", 0) == 0
    assert L.trn_error_name(9001) == b"TRN_ERROR_WAIT_ABANDONED"
    # a list is validated as a whole before the device is touched: the bad entry is the LAST one
    good = _ffi.GemvDesc(4, 256, 0, 0, 16, 16, 16, 0, 0, 0, 0.0, 0)     # n = 0: a no-op entry
    bad = _ffi.GemvDesc(4, 100, 4, 0, 16, 16, 16, 0, 0, 0, 0.0, 0)      # k % 256 != 0
    assert L.trn_kquant_gemv_batch(None, (_ffi.GemvDesc * 2)(good, bad), 2) == 1
    null_y = _ffi.GemvDesc(4, 256, 4, 0, 0, 16, 16, 0, 0, 0, 0.0, 0)
    assert L.trn_kquant_gemv_batch(None, (_ffi.GemvDesc * 2)(good, null_y), 2) == 1
