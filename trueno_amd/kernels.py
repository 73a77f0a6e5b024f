"""Host mirror of the k-quant kernel types of trueno-gpu/src/kernels/quantize.rs.

Constructors, field names, `name()` strings and kernel parameter order are the reference's.
`emit_ptx/build_ptx/as_module` (kernels/mod.rs:47-102) have no meaning without a PTX backend;
their place is taken by `launch_config()` (the reference's documented geometry, kept for callers
that build a LaunchConfig themselves - the library substitutes the kernel's real geometry) and
`launch()` (the typed C-ABI launcher).
"""
from __future__ import annotations

import ctypes as C
import enum

from . import _ffi
from .driver import CudaModule, CudaStream, GpuBuffer, GpuError, LaunchConfig, _check, _lib

# quantize.rs:34-53
Q4K_BLOCK_SIZE = 32
Q4K_SUPER_BLOCK_SIZE = 256
Q4K_SUPER_BLOCK_BYTES = 144
Q4K_BLOCK_BYTES = 18
Q5K_SUPER_BLOCK_SIZE = 256
Q5K_SUPER_BLOCK_BYTES = 176
Q6K_SUPER_BLOCK_SIZE = 256
Q6K_SUPER_BLOCK_BYTES = 210


class Q4KFormat(enum.Enum):
    """quantize.rs:56-62."""
    Simplified = 0
    GgmlSuperBlock = 1


class Kernel:
    """kernels/mod.rs:47-102 (the part that survives without PTX)."""

    def name(self) -> str:
        raise NotImplementedError

    def launch_config(self) -> LaunchConfig:
        raise NotImplementedError


def _ptr(b) -> int:
    return b.as_ptr() if isinstance(b, GpuBuffer) else int(b)


class _GemvKernel(Kernel):
    _NAME = ""
    _SB_BYTES = 0
    _LAUNCHER = ""

    def __init__(self, k: int, n: int):
        """k first, then n (quantize.rs:1171-1173)."""
        self.k = int(k)
        self.n = int(n)

    def name(self) -> str:
        return self._NAME

    def num_super_blocks_per_row(self) -> int:
        return self.k // 256

    def weight_bytes(self) -> int:
        return self.n * self.num_super_blocks_per_row() * self._SB_BYTES

    def launch_config(self) -> LaunchConfig:
        """grid = N blocks, block = 32 threads, no shared memory (quantize.rs:1151-1155)."""
        return LaunchConfig((self.n, 1, 1), (32, 1, 1), 0)

    def kernel_args(self, y, w, x):
        """(y_ptr, w_ptr, x_ptr, k_dim, n_dim) - quantize.rs:1190-1194."""
        return [C.c_uint64(_ptr(y)), C.c_uint64(_ptr(w)), C.c_uint64(_ptr(x)), C.c_uint32(self.k), C.c_uint32(self.n)]

    def launch(self, stream: CudaStream, y, w, x) -> None:
        fn = getattr(_lib(), self._LAUNCHER)
        _check(fn(stream.raw() if stream is not None else None, _ptr(y), _ptr(w), _ptr(x), self.k, self.n),
               "KernelLaunch", self._NAME)

    def launch_by_name(self, stream: CudaStream, module: CudaModule, y, w, x) -> None:
        """The reference's call shape: launch_kernel(module, name, LaunchConfig, args)."""
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(y, w, x))


class Q4KGemvKernel(_GemvKernel):
    """quantize.rs:1156-1523."""
    _NAME = "q4k_gemv_warp_reduce"
    _SB_BYTES = Q4K_SUPER_BLOCK_BYTES
    _LAUNCHER = "trn_q4k_gemv"


class Q5KGemvKernel(_GemvKernel):
    """quantize.rs:1532-1724."""
    _NAME = "q5k_gemv_warp_reduce"
    _SB_BYTES = Q5K_SUPER_BLOCK_BYTES
    _LAUNCHER = "trn_q5k_gemv"


class Q6KGemvKernel(_GemvKernel):
    """quantize.rs:1733-1965."""
    _NAME = "q6k_gemv_warp_reduce"
    _SB_BYTES = Q6K_SUPER_BLOCK_BYTES
    _LAUNCHER = "trn_q6k_gemv"


class _GemmKernel(Kernel):
    _NAME = ""
    _SB_BYTES = 0
    _LAUNCHER = ""

    def __init__(self, m: int, n: int, k: int):
        self.m, self.n, self.k = int(m), int(n), int(k)
        self.tile_size = 32

    def name(self) -> str:
        return self._NAME

    def with_tile_size(self, tile_size: int):
        self.tile_size = int(tile_size)
        return self

    def num_super_blocks_per_row(self) -> int:
        return self.k // 256

    def weight_bytes(self) -> int:
        return self.n * self.num_super_blocks_per_row() * self._SB_BYTES

    def launch_config(self) -> LaunchConfig:
        """tile_size^2 threads per block, one block per output tile (quantize.rs:376-386)."""
        t = self.tile_size
        return LaunchConfig(((self.n + t - 1) // t, (self.m + t - 1) // t, 1), (t * t, 1, 1), 0)

    def kernel_args(self, a, b_quant, c):
        """(a_ptr, b_quant_ptr, c_ptr, m, n, k) - quantize.rs:354-359."""
        return [C.c_uint64(_ptr(a)), C.c_uint64(_ptr(b_quant)), C.c_uint64(_ptr(c)),
                C.c_uint32(self.m), C.c_uint32(self.n), C.c_uint32(self.k)]

    def launch(self, stream: CudaStream, a, b_quant, c, as_written: bool = False) -> None:
        """as_written: the weights decoded as the reference's GEMM kernels write it (quantize.rs:445-514, :727-807,
        :1009-1064) instead of the canonical decode the GEMV kernels share."""
        fn = getattr(_lib(), self._LAUNCHER + ("_as_written" if as_written else ""))
        _check(fn(stream.raw() if stream is not None else None, _ptr(a), _ptr(b_quant), _ptr(c), self.m, self.n, self.k),
               "KernelLaunch", self._NAME)

    def launch_by_name(self, stream: CudaStream, module: CudaModule, a, b_quant, c) -> None:
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(a, b_quant, c))


class QuantizeKernel(_GemmKernel):
    """quantize.rs:66-147.  `QuantizeKernel.ggml(m, n, k)` is the 144-byte super-block format
    (q4k_gemm_ggml); the plain constructor is the legacy "simplified" format of 18-byte blocks of 32
    values (q4k_gemm_fused, quantize.rs:84-93, 151-336)."""
    _SB_BYTES = Q4K_SUPER_BLOCK_BYTES
    _LAUNCHER = "trn_q4k_gemm"

    def __init__(self, m: int, n: int, k: int):
        super().__init__(m, n, k)
        self.block_size = Q4K_BLOCK_SIZE
        self.format = Q4KFormat.Simplified

    @staticmethod
    def ggml(m: int, n: int, k: int) -> "QuantizeKernel":
        kern = QuantizeKernel(m, n, k)
        kern.block_size = Q4K_SUPER_BLOCK_SIZE
        kern.format = Q4KFormat.GgmlSuperBlock
        return kern

    def name(self) -> str:
        return "q4k_gemm_ggml" if self.format is Q4KFormat.GgmlSuperBlock else "q4k_gemm_fused"

    def num_blocks_per_row(self) -> int:
        return self.k // self.block_size

    def weight_bytes(self) -> int:
        if self.format is Q4KFormat.GgmlSuperBlock:
            return super().weight_bytes()
        return self.n * self.num_blocks_per_row() * Q4K_BLOCK_BYTES

    def launch(self, stream, a, b_quant, c, as_written: bool = False) -> None:
        if self.format is Q4KFormat.GgmlSuperBlock:
            return super().launch(stream, a, b_quant, c, as_written)
        _check(_lib().trn_q4k_gemm_fused(stream.raw() if stream is not None else None, _ptr(a), _ptr(b_quant), _ptr(c),
                                         self.m, self.n, self.k), "KernelLaunch", self.name())


class Q5KKernel(_GemmKernel):
    """quantize.rs:598-866."""
    _NAME = "q5k_gemm_ggml"
    _SB_BYTES = Q5K_SUPER_BLOCK_BYTES
    _LAUNCHER = "trn_q5k_gemm"


class Q6KKernel(_GemmKernel):
    """quantize.rs:884-1121."""
    _NAME = "q6k_gemm_ggml"
    _SB_BYTES = Q6K_SUPER_BLOCK_BYTES
    _LAUNCHER = "trn_q6k_gemm"


def dequant_simplified_f32(stream: CudaStream, out, w, n_blocks: int) -> None:
    """Test surface: out[b*32+i] = weight i of 18-byte simplified block b (quantize.rs:237-267)."""
    _check(_lib().trn_q4k_simplified_dequant_f32(stream.raw() if stream is not None else None, _ptr(out), _ptr(w), int(n_blocks)),
           "KernelLaunch", "q4k_simplified_dequant_f32")


def dequant_f32(fmt: str, stream: CudaStream, out, w, n_sb: int, policy: int = 0) -> None:
    """Test surface: out[sb*256+i] = weight i of super-block sb (policy 0 GEMV family, 1 GEMM family)."""
    fn = getattr(_lib(), f"trn_{fmt}_dequant_f32")
    _check(fn(stream.raw() if stream is not None else None, _ptr(out), _ptr(w), int(n_sb), int(policy)),
           "KernelLaunch", f"{fmt}_dequant_f32")


class GemvBatch:
    """An ordered list of k-quant GEMVs issued with one library call (trn_kquant_gemv_batch): the
    weight pass of one decode step.  Entries run in order on the stream; a later entry may read an
    earlier entry's output."""

    _FMT = {"q4k": 4, "q5k": 5, "q6k": 6}

    def __init__(self):
        self._entries = []
        self._array = None

    NORM_INPUT = 1    # the entry reads x / sqrt(mean(x^2) + eps) instead of x
    SWIGLU_INPUT = 8  # the entry reads silu(x) * x2 instead of x (x = gate, x2 = up)

    def add(self, fmt: str, k: int, n: int, y, w, x, flags: int = 0, gamma=None, x2=None, residual=None,
            norm_eps: float = 0.0) -> "GemvBatch":
        """y = s * W (x' * gamma) + residual with x' = x or silu(x) * x2 and s = 1 or the RMS normalisation of x':
        the element-wise steps of a decoder layer (rmsnorm, fused_swiglu, residual_add) folded into the GEMV."""
        if x2 is not None:
            flags |= self.SWIGLU_INPUT
        self._entries.append(_ffi.GemvDesc(self._FMT[fmt], int(k), int(n), int(flags), _ptr(y), _ptr(w), _ptr(x),
                                           0 if gamma is None else _ptr(gamma), 0 if x2 is None else _ptr(x2),
                                           0 if residual is None else _ptr(residual), float(norm_eps), 0))
        self._array = None
        return self

    def __len__(self) -> int:
        return len(self._entries)

    def plan(self):
        """launch_of[i]: which launch (0, 1, ... in launch order) the library's default mode puts entry i into.
        Launches nothing."""
        import ctypes as C
        if self._array is None:
            self._array = (_ffi.GemvDesc * len(self._entries))(*self._entries)
        out = (C.c_uint32 * len(self._entries))()
        _check(_lib().trn_kquant_gemv_plan(self._array, len(self._entries), out), "KernelLaunch", "kquant_gemv_plan")
        return list(out)

    def subset(self, indices) -> "GemvBatch":
        """A list of the given entries of this one, in the given order."""
        b = GemvBatch()
        b._entries = [self._entries[i] for i in indices]
        return b

    def launch(self, stream: CudaStream) -> None:
        if self._array is None:
            self._array = (_ffi.GemvDesc * len(self._entries))(*self._entries)
        _check(_lib().trn_kquant_gemv_batch(stream.raw() if stream is not None else None, self._array, len(self._entries)),
               "KernelLaunch", "kquant_gemv_batch")
