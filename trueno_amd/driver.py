"""Host mirror of trueno_gpu::driver for the k-quant path, over libtrueno_hip.so.

Same names, argument meaning and error behaviour as the reference's safe wrappers:
  CudaContext   trueno-gpu/src/driver/context.rs:97-239
  CudaModule    trueno-gpu/src/driver/module.rs:62-144   (from_ptx becomes from_builtin/from_image)
  CudaStream    trueno-gpu/src/driver/stream.rs:55-166
  GpuBuffer     trueno-gpu/src/driver/memory.rs:66-683
  LaunchConfig  trueno-gpu/src/driver/types.rs:86-142
  GpuError      trueno-gpu/src/error.rs:41-107  (`kind` carries the Rust variant name)
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass
from typing import Optional, Sequence, Tuple

import numpy as np

from . import _ffi


class GpuError(Exception):
    """kind is the reference's GpuError variant: CudaDriver, MemoryAllocation, KernelLaunch, DeviceInit,
    DeviceNotFound, ModuleLoad, FunctionNotFound, StreamCreate, StreamSync, Transfer, CudaNotAvailable."""

    def __init__(self, kind: str, message: str, code: int = 0):
        super().__init__(f"{kind}: {message}")
        self.kind = kind
        self.message = message
        self.code = code


_NO_DEVICE = 100


def _lib():
    try:
        return _ffi.lib()
    except OSError as e:  # missing library == no driver (driver/sys.rs:373-391)
        raise GpuError("CudaNotAvailable", str(e)) from e


def _check(code: int, kind: str, what: str = "") -> None:
    """sys.rs:360-369 maps a non-zero result to CudaDriver(name, code); call sites re-map it."""
    if code == 0:
        return
    L = _lib()
    name = (L.trn_error_name(code) or b"?").decode()
    text = (L.trn_error_string(code) or b"?").decode()
    if code == _NO_DEVICE:
        raise GpuError("CudaNotAvailable", f"{name}: {text}", code)
    raise GpuError(kind, f"{what + ': ' if what else ''}{name} (code: {code}): {text}", code)


def cuda_available() -> bool:
    """driver/mod.rs:89-101: true when the driver loads and a device exists."""
    try:
        return device_count() > 0
    except GpuError:
        return False


def device_count() -> int:
    L = _lib()
    _check(L.trn_init(0), "DeviceInit", "init")
    n = C.c_int(0)
    _check(L.trn_device_get_count(C.byref(n)), "DeviceInit", "device count")
    return int(n.value)


class CudaContext:
    """Primary context of one device (context.rs:97-135).  Made current on the creating thread."""

    def __init__(self, device_ordinal: int = 0):
        L = _lib()
        _check(L.trn_init(0), "DeviceInit", "init")
        n = C.c_int(0)
        _check(L.trn_device_get_count(C.byref(n)), "DeviceInit", "device count")
        if device_ordinal < 0 or device_ordinal >= n.value:
            raise GpuError("DeviceNotFound", f"CUDA device {device_ordinal} not found (available: {n.value})")
        dev = C.c_int(0)
        _check(L.trn_device_get(C.byref(dev), device_ordinal), "DeviceInit", "device get")
        ctx = C.c_void_p()
        _check(L.trn_primary_ctx_retain(C.byref(ctx), dev.value), "DeviceInit", "primary context")
        _check(L.trn_ctx_set_current(ctx), "DeviceInit", "set current")
        self._dev = dev.value
        self._ctx = ctx
        self._released = False

    def device(self) -> int:
        return self._dev

    def make_current(self) -> None:
        _check(_lib().trn_ctx_set_current(self._ctx), "DeviceInit", "set current")

    def memory_info(self) -> Tuple[int, int]:
        free, total = C.c_size_t(0), C.c_size_t(0)
        _check(_lib().trn_mem_get_info(C.byref(free), C.byref(total)), "CudaDriver", "mem info")
        return int(free.value), int(total.value)

    def synchronize(self) -> None:
        _check(_lib().trn_ctx_synchronize(), "StreamSync", "context synchronize")

    def device_name(self) -> str:
        buf = C.create_string_buffer(256)
        _check(_lib().trn_device_get_name(buf, 256, self._dev), "DeviceInit", "device name")
        return buf.value.decode()

    def total_memory(self) -> int:
        n = C.c_size_t(0)
        _check(_lib().trn_device_total_mem(C.byref(n), self._dev), "DeviceInit", "total memory")
        return int(n.value)

    def cu_count(self) -> int:
        n = C.c_int(0)
        _check(_lib().trn_device_cu_count(C.byref(n)), "CudaDriver", "cu count")
        return int(n.value)

    def release(self) -> None:
        if not self._released:
            self._released = True
            _lib().trn_primary_ctx_release(self._dev)

    def __del__(self):
        try:
            self.release()
        except Exception:
            pass


@dataclass(frozen=True)
class LaunchConfig:
    """types.rs:86-142."""
    grid: Tuple[int, int, int] = (1, 1, 1)
    block: Tuple[int, int, int] = (256, 1, 1)
    shared_mem: int = 0

    @staticmethod
    def linear(num_elements: int, block_size: int) -> "LaunchConfig":
        return LaunchConfig(((num_elements + block_size - 1) // block_size, 1, 1), (block_size, 1, 1), 0)

    @staticmethod
    def grid_2d(grid_x: int, grid_y: int, block_x: int, block_y: int) -> "LaunchConfig":
        return LaunchConfig((grid_x, grid_y, 1), (block_x, block_y, 1), 0)

    def with_shared_mem(self, nbytes: int) -> "LaunchConfig":
        return LaunchConfig(self.grid, self.block, nbytes)

    def total_threads(self) -> int:
        g, b = self.grid, self.block
        return g[0] * g[1] * g[2] * b[0] * b[1] * b[2]


class CudaModule:
    """A loaded code object (module.rs:62-144).  `from_builtin` stands where the reference does
    from_ptx(ctx, kernel.emit_ptx()): the k-quant kernels ship precompiled for gfx950."""

    def __init__(self, handle: C.c_void_p):
        self._h = handle
        self._functions = {}

    @staticmethod
    def from_builtin(ctx: CudaContext) -> "CudaModule":
        ctx.make_current()
        h = C.c_void_p()
        _check(_lib().trn_module_load_builtin(C.byref(h)), "ModuleLoad", "built-in code object")
        return CudaModule(h)

    @staticmethod
    def from_image(ctx: CudaContext, image: bytes) -> "CudaModule":
        ctx.make_current()
        if not image:
            raise GpuError("ModuleLoad", "empty code object")
        buf = C.create_string_buffer(image, len(image))
        h = C.c_void_p()
        _check(_lib().trn_module_load_data(C.byref(h), C.cast(buf, C.c_void_p)), "ModuleLoad", "code object")
        return CudaModule(h)

    def get_function(self, name: str) -> C.c_void_p:
        if "\0" in name:
            raise GpuError("FunctionNotFound", name.replace("\0", "\\0"))  # module.rs:99-100
        if name not in self._functions:
            f = C.c_void_p()
            code = _lib().trn_module_get_function(C.byref(f), self._h, name.encode())
            if code != 0:
                raise GpuError("FunctionNotFound", f"CUDA function '{name}' not found in module", code)
            self._functions[name] = f
        return self._functions[name]

    def has_function(self, name: str) -> bool:
        return name in self._functions

    def cached_functions(self):
        return list(self._functions)

    def unload(self) -> None:
        if self._h:
            _lib().trn_module_unload(self._h)
            self._h = None

    def __del__(self):
        try:
            self.unload()
        except Exception:
            pass


class CudaStream:
    """stream.rs:55-166.  Non-blocking stream, default priority."""

    def __init__(self, ctx: CudaContext):
        ctx.make_current()
        s = C.c_void_p()
        _check(_lib().trn_stream_create(C.byref(s), 1), "StreamCreate")
        self._s = s

    def raw(self) -> C.c_void_p:
        return self._s

    def synchronize(self) -> None:
        _check(_lib().trn_stream_synchronize(self._s), "StreamSync")

    def launch_kernel(self, module: CudaModule, func_name: str, config: LaunchConfig, args: Sequence) -> None:
        """args: ctypes scalars in the kernel's declared parameter order (stream.rs:110-154)."""
        fn = module.get_function(func_name)
        holders = list(args)
        arr = (C.c_void_p * len(holders))(*[C.cast(C.pointer(a), C.c_void_p) for a in holders])
        g, b = config.grid, config.block
        code = _lib().trn_launch_kernel(fn, g[0], g[1], g[2], b[0], b[1], b[2], config.shared_mem, self._s, arr, None)
        _check(code, "KernelLaunch", func_name)

    def destroy(self) -> None:
        if self._s:
            _lib().trn_stream_destroy(self._s)
            self._s = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass


class GpuBuffer:
    """Typed device buffer (memory.rs:66-683).  Owns its allocation unless made by from_raw_parts."""

    def __init__(self, ctx: Optional[CudaContext], length: int, dtype=np.float32, _ptr: Optional[int] = None):
        self.dtype = np.dtype(dtype)
        self._len = int(length)
        self._owned = _ptr is None
        self._ptr = 0
        if _ptr is not None:
            self._ptr = int(_ptr)
        elif self._len > 0:  # zero-length: null pointer, no driver call (memory.rs:101-107)
            p = C.c_uint64(0)
            _check(_lib().trn_mem_alloc(C.byref(p), self.size_bytes()), "MemoryAllocation")
            self._ptr = int(p.value)

    @staticmethod
    def from_host(ctx: CudaContext, data: np.ndarray) -> "GpuBuffer":
        data = np.ascontiguousarray(data)
        buf = GpuBuffer(ctx, data.size, data.dtype)
        buf.copy_from_host(data)
        return buf

    @staticmethod
    def from_raw_parts(ptr: int, length: int, dtype=np.float32) -> "GpuBuffer":
        return GpuBuffer(None, length, dtype, _ptr=ptr)

    def clone_metadata(self) -> "GpuBufferView":
        """A view of the same device memory that owns nothing (memory.rs:148-170)."""
        return GpuBufferView(self._ptr, self._len, self.dtype)

    def as_ptr(self) -> int:
        return self._ptr

    def as_kernel_arg(self) -> C.c_uint64:
        return C.c_uint64(self._ptr)

    def len(self) -> int:
        return self._len

    def __len__(self) -> int:
        return self._len

    def is_empty(self) -> bool:
        return self._len == 0

    def size_bytes(self) -> int:
        return self._len * self.dtype.itemsize

    def _host(self, data) -> np.ndarray:
        a = np.ascontiguousarray(data, dtype=self.dtype).reshape(-1)
        return a

    def copy_from_host(self, data) -> None:
        a = self._host(data)
        if a.size != self._len:  # memory.rs:221-227
            raise GpuError("Transfer", f"Length mismatch: host {a.size} vs device {self._len}")
        if self._len == 0:
            return
        _check(_lib().trn_memcpy_htod(self._ptr, a.ctypes.data, a.nbytes), "Transfer")

    def copy_to_host(self, out: Optional[np.ndarray] = None) -> np.ndarray:
        if out is None:
            out = np.empty(self._len, self.dtype)
        if out.size != self._len or out.dtype != self.dtype or not out.flags.c_contiguous:
            raise GpuError("Transfer", f"Length mismatch: host {out.size} vs device {self._len}")
        if self._len:
            _check(_lib().trn_memcpy_dtoh(out.ctypes.data, self._ptr, out.nbytes), "Transfer")
        return out

    def copy_from_host_at(self, data, offset: int) -> None:
        a = self._host(data)
        if offset + a.size > self._len:  # memory.rs:388-396
            raise GpuError("Transfer", f"Partial copy out of bounds: offset {offset} + len {a.size} > buffer {self._len}")
        if a.size == 0:
            return
        _check(_lib().trn_memcpy_htod(self._ptr + offset * self.dtype.itemsize, a.ctypes.data, a.nbytes), "Transfer")

    def copy_to_host_at(self, out: np.ndarray, offset: int) -> np.ndarray:
        if offset + out.size > self._len:
            raise GpuError("Transfer", f"Partial copy out of bounds: offset {offset} + len {out.size} > buffer {self._len}")
        if out.size:
            _check(_lib().trn_memcpy_dtoh(out.ctypes.data, self._ptr + offset * self.dtype.itemsize, out.nbytes), "Transfer")
        return out

    def copy_from_host_async(self, data: np.ndarray, stream: CudaStream) -> None:
        """The host array must stay alive and unchanged until the stream reaches the copy (memory.rs:280-312)."""
        if data.size != self._len:
            raise GpuError("Transfer", f"Length mismatch: host {data.size} vs device {self._len}")
        if self._len:
            _check(_lib().trn_memcpy_htod_async(self._ptr, data.ctypes.data, data.nbytes, stream.raw()), "Transfer")

    def copy_to_host_async(self, out: np.ndarray, stream: CudaStream) -> None:
        if out.size != self._len:
            raise GpuError("Transfer", f"Length mismatch: host {out.size} vs device {self._len}")
        if self._len:
            _check(_lib().trn_memcpy_dtoh_async(out.ctypes.data, self._ptr, out.nbytes, stream.raw()), "Transfer")

    def copy_from_buffer(self, src: "GpuBuffer") -> None:
        if src._len != self._len:
            raise GpuError("Transfer", f"Length mismatch: source {src._len} vs destination {self._len}")
        if self._len:
            _check(_lib().trn_memcpy_dtod(self._ptr, src._ptr, self.size_bytes()), "Transfer")

    def copy_from_buffer_async(self, src: "GpuBuffer", stream: CudaStream) -> None:
        if src._len != self._len:
            raise GpuError("Transfer", f"Length mismatch: source {src._len} vs destination {self._len}")
        if self._len:
            _check(_lib().trn_memcpy_dtod_async(self._ptr, src._ptr, self.size_bytes(), stream.raw()), "Transfer")

    def copy_from_buffer_at(self, src: "GpuBuffer", dst_offset: int, src_offset: int, count: int) -> None:
        if dst_offset + count > self._len or src_offset + count > src._len:
            raise GpuError("Transfer", "Partial copy out of bounds")
        if count:
            it = self.dtype.itemsize
            _check(_lib().trn_memcpy_dtod(self._ptr + dst_offset * it, src._ptr + src_offset * it, count * it), "Transfer")

    def copy_from_buffer_at_async(self, src: "GpuBuffer", dst_offset: int, src_offset: int, count: int, stream: CudaStream) -> None:
        """memory.rs:574-611: both buffers must stay valid until the stream has been synchronised."""
        self.copy_from_buffer_at_async_raw(src, dst_offset, src_offset, count, stream.raw())

    def copy_from_buffer_at_async_raw(self, src: "GpuBuffer", dst_offset: int, src_offset: int, count: int, stream_handle) -> None:
        """memory.rs:613-650: the same with the raw stream handle."""
        if dst_offset + count > self._len:
            raise GpuError("Transfer", f"Async D2D dst out of bounds: {dst_offset} + {count} > {self._len}")
        if src_offset + count > src._len:
            raise GpuError("Transfer", f"Async D2D src out of bounds: {src_offset} + {count} > {src._len}")
        if count:
            it = self.dtype.itemsize
            _check(_lib().trn_memcpy_dtod_async(self._ptr + dst_offset * it, src._ptr + src_offset * it, count * it, stream_handle), "Transfer")

    def free(self) -> None:
        if self._owned and self._ptr:
            _lib().trn_mem_free(self._ptr)
        self._ptr = 0
        self._len = 0

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class GpuBufferView:
    """Non-owning view of a device buffer (memory.rs:172-207): a pointer and a length, nothing is freed with it."""

    def __init__(self, ptr: int, length: int, dtype=np.float32):
        self._ptr, self._len, self.dtype = int(ptr), int(length), np.dtype(dtype)

    def as_ptr(self) -> int:
        return self._ptr

    def len(self) -> int:
        return self._len

    def __len__(self) -> int:
        return self._len

    def is_empty(self) -> bool:
        return self._len == 0

    def size_bytes(self) -> int:
        return self._len * self.dtype.itemsize
