"""The Rust binding under rust/trueno-gpu-hip is source only (no Rust toolchain in this image): these checks keep it
in step with the C header it binds - every exported function declared with the same number of parameters, the
constants with the same values, trn_gemv_desc with the same fields in the same order, and the CudaDriver table of
`src/sys.rs` holding the reference's 25 `cu*` fields (trueno-gpu/src/driver/sys.rs:99-201), each loaded from its
`trn_*` symbol."""
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = open(os.path.join(ROOT, "include", "trueno_hip.h")).read()
FFI = open(os.path.join(ROOT, "rust", "trueno-gpu-hip", "src", "ffi.rs")).read()
SYS = open(os.path.join(ROOT, "rust", "trueno-gpu-hip", "src", "sys.rs")).read()
KERNELS = open(os.path.join(ROOT, "rust", "trueno-gpu-hip", "src", "kernels.rs")).read()


def _strip_comments(text: str) -> str:
    return re.sub(r"/\*.*?\*/", " ", text, flags=re.S)


def _c_functions():
    """{name: parameter count} of the header's TRN_API declarations"""
    out = {}
    for m in re.finditer(r"TRN_API\s+[\w\s\*]+?\b(trn_\w+)\s*\(([^;]*?)\)\s*;", _strip_comments(HEADER), flags=re.S):
        params = m.group(2).strip()
        out[m.group(1)] = 0 if params in ("", "void") else params.count(",") + 1
    return out


def _rust_functions():
    out = {}
    for m in re.finditer(r"pub fn (trn_\w+)\s*\(([^;]*?)\)\s*(?:->[^;]+)?;", FFI, flags=re.S):
        params = [p for p in m.group(2).split(",") if p.strip()]
        out[m.group(1)] = len(params)
    return out


def test_every_entry_point_is_declared_with_the_same_arity():
    c, r = _c_functions(), _rust_functions()
    assert len(c) >= 60
    assert set(c) == set(r), (sorted(set(c) - set(r)), sorted(set(r) - set(c)))
    assert {n: c[n] for n in c} == {n: r[n] for n in c}


def test_constants_agree():
    for name, value in re.findall(r"#define (TRN_[A-Z_]+) (\d+)u?\b", HEADER):
        if name == "TRN_API":
            continue
        m = re.search(rf"pub const {name}: [\w:]+ = (\d+);", FFI)
        assert m, name
        assert int(m.group(1)) == int(value), name


def test_gemv_desc_layout():
    body = re.search(r"typedef struct trn_gemv_desc \{(.*?)\} trn_gemv_desc;", HEADER, flags=re.S).group(1)
    c_fields = re.findall(r"(\w+)\s+(\w+);", _strip_comments(body))
    body = re.search(r"pub struct trn_gemv_desc \{(.*?)\n\}", FFI, flags=re.S).group(1)
    r_fields = re.findall(r"pub (\w+): (\w+),", body)
    ctype = {"uint32_t": "u32", "trn_dptr": "trn_dptr", "float": "f32"}
    assert [(n, ctype[t]) for t, n in c_fields] == r_fields
    assert "#[repr(C)]" in FFI.split("pub struct trn_gemv_desc")[0][-80:]


# the reference's table, in its order, and the symbol that fills each field
DRIVER_TABLE = [
    ("cuInit", "trn_init"), ("cuDeviceGetCount", "trn_device_get_count"), ("cuDeviceGet", "trn_device_get"),
    ("cuDeviceGetName", "trn_device_get_name"), ("cuDeviceTotalMem", "trn_device_total_mem"),
    ("cuDevicePrimaryCtxRetain", "trn_primary_ctx_retain"), ("cuDevicePrimaryCtxRelease", "trn_primary_ctx_release"),
    ("cuCtxSetCurrent", "trn_ctx_set_current"), ("cuCtxSynchronize", "trn_ctx_synchronize"),
    ("cuModuleLoadData", "trn_module_load_data"), ("cuModuleUnload", "trn_module_unload"),
    ("cuModuleGetFunction", "trn_module_get_function"), ("cuMemAlloc", "trn_mem_alloc"), ("cuMemFree", "trn_mem_free"),
    ("cuMemcpyHtoD", "trn_memcpy_htod"), ("cuMemcpyDtoH", "trn_memcpy_dtoh"), ("cuMemcpyHtoDAsync", "trn_memcpy_htod_async"),
    ("cuMemcpyDtoHAsync", "trn_memcpy_dtoh_async"), ("cuMemcpyDtoD", "trn_memcpy_dtod"),
    ("cuMemcpyDtoDAsync", "trn_memcpy_dtod_async"), ("cuMemGetInfo", "trn_mem_get_info"),
    ("cuStreamCreate", "trn_stream_create"), ("cuStreamDestroy", "trn_stream_destroy"),
    ("cuStreamSynchronize", "trn_stream_synchronize"), ("cuLaunchKernel", "trn_launch_kernel"),
]


def test_driver_table_holds_the_reference_fields_and_binds_exported_symbols():
    assert len(DRIVER_TABLE) == 25
    for field, symbol in DRIVER_TABLE:
        assert re.search(rf"pub {field}:\s*unsafe extern \"C\" fn", SYS), field
        assert re.search(rf"{field}: sym!\(b\"{symbol}\\0\"\)", SYS), (field, symbol)
    exported = _c_functions()
    for symbol in re.findall(r"sym!\(b\"(trn_\w+)\\0\"\)", SYS):
        assert symbol in exported, symbol


def test_kernel_names_and_sizes_are_the_reference_ones():
    from trueno_amd import kernels as K
    for const in ("Q4K_BLOCK_SIZE", "Q4K_SUPER_BLOCK_SIZE", "Q4K_SUPER_BLOCK_BYTES", "Q4K_BLOCK_BYTES", "Q5K_SUPER_BLOCK_SIZE",
                  "Q5K_SUPER_BLOCK_BYTES", "Q6K_SUPER_BLOCK_SIZE", "Q6K_SUPER_BLOCK_BYTES"):
        m = re.search(rf"pub const {const}: u32 = (\d+);", KERNELS)
        assert m and int(m.group(1)) == getattr(K, const), const
    for cls, args in ((K.Q4KGemvKernel, (256, 1)), (K.Q5KGemvKernel, (256, 1)), (K.Q6KGemvKernel, (256, 1)),
                      (K.Q5KKernel, (1, 1, 256)), (K.Q6KKernel, (1, 1, 256)), (K.QuantizeKernel, (1, 1, 256))):
        assert f'"{cls(*args).name()}"' in KERNELS, cls.__name__
    assert '"q4k_gemm_ggml"' in KERNELS
