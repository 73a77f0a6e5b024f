"""trueno_amd: MI355X (gfx950) backend for trueno-gpu's fused k-quant matrix path.

Host-side mirror of the trueno-gpu surface for this path (same type, method and kernel names)
over the C ABI of libtrueno_hip.so:

    trueno_amd.driver   CudaContext, CudaModule, CudaStream, GpuBuffer, GpuBufferView, LaunchConfig, GpuError
                        (trueno-gpu/src/driver/{context,module,stream,memory,types}.rs, src/error.rs)
    trueno_amd.kernels  Kernel, Q4KGemvKernel, Q5KGemvKernel, Q6KGemvKernel, QuantizeKernel,
                        Q5KKernel, Q6KKernel, Q4KFormat   (trueno-gpu/src/kernels/quantize.rs)
    trueno_amd.glue     ResidualAddKernel, FusedSwigluKernel, RmsNormKernel, FusedResidualRmsNormKernel, GemvKernel,
                        CoalescedGemvKernel, IncrementalAttentionKernel
                        (trueno-gpu/src/kernels/elementwise.rs, layernorm.rs, gemv.rs, attention.rs)

There is no CPU path: without libtrueno_hip.so or without a GPU every device call raises GpuError.
"""
from . import _ffi  # noqa: F401
from .driver import (CudaContext, CudaModule, CudaStream, GpuBuffer, GpuBufferView, GpuError, LaunchConfig,  # noqa: F401
                     cuda_available, device_count)
from .kernels import (GemvBatch, Kernel, Q4KFormat, Q4KGemvKernel, Q5KGemvKernel, Q5KKernel, Q6KGemvKernel,  # noqa: F401
                      Q6KKernel, QuantizeKernel)
from .glue import (CoalescedGemvKernel, FusedResidualRmsNormKernel, FusedSwigluKernel, GemvKernel,  # noqa: F401
                   IncrementalAttentionKernel, ResidualAddKernel, RmsNormKernel)
