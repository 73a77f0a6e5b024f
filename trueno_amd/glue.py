"""Host mirror of the element-wise decoder-layer kernels of trueno-gpu (kernels/elementwise.rs, kernels/layernorm.rs):
ResidualAddKernel, FusedSwigluKernel, RmsNormKernel, FusedResidualRmsNormKernel - and of its f32 GEMV kernels
(kernels/gemv.rs): GemvKernel, CoalescedGemvKernel.

Constructors, fields, `name()` strings and parameter lists are the reference's.  The reference compiles
`hidden_size` and `epsilon` of the two norms (and the shape of the attention kernel) into the PTX of one kernel
instance; with a pre-built code object they are constants of the function handle, which `launch_by_name()` sets
(trn_function_set_rmsnorm / trn_function_set_attention) before it launches with the reference's own arguments.
"""
from __future__ import annotations

import ctypes as C

from .driver import CudaModule, CudaStream, LaunchConfig, _check, _lib
from .kernels import Kernel, _ptr


class ResidualAddKernel(Kernel):
    """output = input1 + input2 (elementwise.rs:33-101)."""

    def __init__(self, n: int):
        self.n = int(n)

    def name(self) -> str:
        return "residual_add"

    def launch_config(self) -> LaunchConfig:
        """block 256, grid ceil(n / 256) (elementwise.rs:27-30)."""
        return LaunchConfig.linear(self.n, 256)

    def kernel_args(self, input1, input2, output):
        return [C.c_uint64(_ptr(input1)), C.c_uint64(_ptr(input2)), C.c_uint64(_ptr(output)), C.c_uint32(self.n)]

    def launch(self, stream: CudaStream, input1, input2, output) -> None:
        _check(_lib().trn_residual_add(stream.raw() if stream is not None else None, _ptr(input1), _ptr(input2),
                                       _ptr(output), self.n), "KernelLaunch", self.name())

    def launch_by_name(self, stream: CudaStream, module: CudaModule, input1, input2, output) -> None:
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(input1, input2, output))


class FusedSwigluKernel(Kernel):
    """output = silu(gate) * up (elementwise.rs:521-592)."""

    def __init__(self, n: int):
        self.n = int(n)

    def name(self) -> str:
        return "fused_swiglu"

    def launch_config(self) -> LaunchConfig:
        return LaunchConfig.linear(self.n, 256)

    def kernel_args(self, gate, up, output):
        return [C.c_uint64(_ptr(gate)), C.c_uint64(_ptr(up)), C.c_uint64(_ptr(output)), C.c_uint32(self.n)]

    def launch(self, stream: CudaStream, gate, up, output) -> None:
        _check(_lib().trn_fused_swiglu(stream.raw() if stream is not None else None, _ptr(gate), _ptr(up), _ptr(output),
                                       self.n), "KernelLaunch", self.name())

    def launch_by_name(self, stream: CudaStream, module: CudaModule, gate, up, output) -> None:
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(gate, up, output))


class RmsNormKernel(Kernel):
    """output = input / sqrt(mean(input^2) + epsilon) * gamma, one row (layernorm.rs:388-516)."""

    def __init__(self, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.epsilon = 1e-5                     # layernorm.rs:400-405

    def with_epsilon(self, epsilon: float) -> "RmsNormKernel":
        self.epsilon = float(epsilon)
        return self

    def name(self) -> str:
        return "rmsnorm"

    def launch_config(self) -> LaunchConfig:
        """one block of one warp (layernorm.rs:421-423)."""
        return LaunchConfig((1, 1, 1), (32, 1, 1), 0)

    def kernel_args(self, input, output, gamma):
        """(input_ptr, output_ptr, gamma_ptr) - layernorm.rs:426-428."""
        return [C.c_uint64(_ptr(input)), C.c_uint64(_ptr(output)), C.c_uint64(_ptr(gamma))]

    def launch(self, stream: CudaStream, input, output, gamma) -> None:
        _check(_lib().trn_rmsnorm(stream.raw() if stream is not None else None, _ptr(input), _ptr(output), _ptr(gamma),
                                  self.hidden_size, self.epsilon), "KernelLaunch", self.name())

    def launch_by_name(self, stream: CudaStream, module: CudaModule, input, output, gamma) -> None:
        _check(_lib().trn_function_set_rmsnorm(module.get_function(self.name()), self.hidden_size, self.epsilon),
               "KernelLaunch", self.name())
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(input, output, gamma))


class FusedResidualRmsNormKernel(Kernel):
    """output = rmsnorm(residual + input, gamma, epsilon), one row (elementwise.rs:109-248)."""

    def __init__(self, hidden_size: int):
        self.hidden_size = int(hidden_size)
        self.epsilon = 1e-5                     # elementwise.rs:119-123

    def with_epsilon(self, epsilon: float) -> "FusedResidualRmsNormKernel":
        self.epsilon = float(epsilon)
        return self

    def name(self) -> str:
        return "fused_residual_rmsnorm"

    def launch_config(self) -> LaunchConfig:
        return LaunchConfig((1, 1, 1), (32, 1, 1), 0)

    def kernel_args(self, residual, input, output, gamma):
        """(residual_ptr, input_ptr, output_ptr, gamma_ptr) - elementwise.rs:146-149."""
        return [C.c_uint64(_ptr(residual)), C.c_uint64(_ptr(input)), C.c_uint64(_ptr(output)), C.c_uint64(_ptr(gamma))]

    def launch(self, stream: CudaStream, residual, input, output, gamma) -> None:
        _check(_lib().trn_fused_residual_rmsnorm(stream.raw() if stream is not None else None, _ptr(residual), _ptr(input),
                                                 _ptr(output), _ptr(gamma), self.hidden_size, self.epsilon),
               "KernelLaunch", self.name())

    def launch_by_name(self, stream: CudaStream, module: CudaModule, residual, input, output, gamma) -> None:
        _check(_lib().trn_function_set_rmsnorm(module.get_function(self.name()), self.hidden_size, self.epsilon),
               "KernelLaunch", self.name())
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(residual, input, output, gamma))


class _GemvF32(Kernel):
    """y = A x-style product with A K x N row-major: y[n] = sum_k A[k][n] x[k] (gemv.rs)."""
    _NAME = ""

    def __init__(self, k: int, n: int):
        self.k = int(k)
        self.n = int(n)

    def name(self) -> str:
        return self._NAME

    def kernel_args(self, y, a, x):
        """(y_ptr, a_ptr, x_ptr, k_dim, n_dim) - gemv.rs:53-57, 222-226."""
        return [C.c_uint64(_ptr(y)), C.c_uint64(_ptr(a)), C.c_uint64(_ptr(x)), C.c_uint32(self.k), C.c_uint32(self.n)]

    def launch(self, stream: CudaStream, y, a, x) -> None:
        _check(_lib().trn_gemv_f32(stream.raw() if stream is not None else None, _ptr(y), _ptr(a), _ptr(x), self.k, self.n),
               "KernelLaunch", self.name())

    def launch_by_name(self, stream: CudaStream, module: CudaModule, y, a, x) -> None:
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(y, a, x))


class GemvKernel(_GemvF32):
    """gemv.rs:21-166: one warp per output element."""
    _NAME = "gemv_warp_reduce"

    def launch_config(self) -> LaunchConfig:
        return LaunchConfig((self.n, 1, 1), (32, 1, 1), 0)


class CoalescedGemvKernel(_GemvF32):
    """gemv.rs:188-398: 256 threads per block, one output element per thread, x tiles of 256 in shared memory."""
    _NAME = "gemv_coalesced"

    def launch_config(self) -> LaunchConfig:
        return LaunchConfig(((self.n + 255) // 256, 1, 1), (256, 1, 1), 1024)


class IncrementalAttentionKernel(Kernel):
    """Single-query attention over a KV cache (attention.rs:808-1095): q, out [num_heads][head_dim];
    k, v [num_kv_heads][max_seq_len][head_dim]."""

    def __init__(self, max_seq_len: int, head_dim: int, num_heads: int):
        self.max_seq_len, self.head_dim, self.num_heads = int(max_seq_len), int(head_dim), int(num_heads)
        self.num_kv_heads = self.num_heads
        self.scale = 1.0 / float(self.head_dim) ** 0.5           # attention.rs:849

    @classmethod
    def with_gqa(cls, max_seq_len: int, head_dim: int, num_heads: int, num_kv_heads: int) -> "IncrementalAttentionKernel":
        k = cls(max_seq_len, head_dim, num_heads)
        k.num_kv_heads = int(num_kv_heads)
        return k

    def is_gqa(self) -> bool:
        return self.num_kv_heads != self.num_heads

    def name(self) -> str:
        return "incremental_attention"

    def launch_config(self) -> LaunchConfig:
        """one warp per query head (attention.rs:871-873)."""
        return LaunchConfig((self.num_heads, 1, 1), (32, 1, 1), 0)

    def kernel_args(self, q, k, v, out, seq_len: int):
        """(q_ptr, k_ptr, v_ptr, out_ptr, seq_len) - attention.rs:897-901."""
        return [C.c_uint64(_ptr(q)), C.c_uint64(_ptr(k)), C.c_uint64(_ptr(v)), C.c_uint64(_ptr(out)), C.c_uint32(seq_len)]

    def launch(self, stream: CudaStream, q, k, v, out, seq_len: int) -> None:
        _check(_lib().trn_incremental_attention(stream.raw() if stream is not None else None, _ptr(q), _ptr(k), _ptr(v), _ptr(out),
                                                int(seq_len), self.head_dim, self.num_heads, self.num_kv_heads, self.max_seq_len,
                                                self.scale), "KernelLaunch", self.name())

    def launch_by_name(self, stream: CudaStream, module: CudaModule, q, k, v, out, seq_len: int) -> None:
        _check(_lib().trn_function_set_attention(module.get_function(self.name()), self.head_dim, self.num_heads,
                                                 self.num_kv_heads, self.max_seq_len, self.scale), "KernelLaunch", self.name())
        stream.launch_kernel(module, self.name(), self.launch_config(), self.kernel_args(q, k, v, out, seq_len))
