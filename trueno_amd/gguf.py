"""GGUF tensor reader for the k-quant path: finds a tensor's bytes in a GGUF file (format version 2 or 3, little endian)
and puts them on the GPU in the layout the kernels read.

Q4_K and Q6_K tensors are uploaded as they lie in the file: trueno-gpu's Q4_K/Q6_K kernels decode GGML's blocks byte for
byte (trueno-gpu/src/kernels/quantize.rs:1306-1309, 1760-1769).  Q5_K tensors are re-packed on the GPU after the upload
(`trn_q5k_from_ggml`): the reference's Q5_K kernels read their own layout (quantize.rs:1589-1693), not GGML's.  F32
tensors (norm weights) are uploaded unchanged.  The file is memory-mapped; nothing else of it is read.

A GGUF tensor's first dimension is the contiguous one: a weight matrix with ne = [K, N] is N rows of K values, i.e. N rows
of K/256 super-blocks - exactly the (n, k) the GEMV kernels take.
"""
from __future__ import annotations

import mmap
import struct
from dataclasses import dataclass
from typing import Dict, Tuple

import numpy as np

from .driver import CudaContext, CudaStream, GpuBuffer, GpuError, _check, _lib

GGUF_MAGIC = 0x46554747          # "GGUF"
GGML_F32, GGML_F16, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 0, 1, 12, 13, 14
# type -> (values per block, bytes per block)
_BLOCK = {GGML_F32: (1, 4), GGML_F16: (1, 2), GGML_Q4_K: (256, 144), GGML_Q5_K: (256, 176), GGML_Q6_K: (256, 210)}
_FMT = {GGML_Q4_K: "q4k", GGML_Q5_K: "q5k", GGML_Q6_K: "q6k"}
_SCALAR = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<?", 10: "<Q", 11: "<q", 12: "<d"}


@dataclass
class TensorInfo:
    name: str
    dims: Tuple[int, ...]     # ne[0] first (the contiguous dimension)
    ggml_type: int
    offset: int               # from the start of the file
    nbytes: int

    @property
    def fmt(self) -> str:
        """'q4k' / 'q5k' / 'q6k' for the k-quant types, else ''."""
        return _FMT.get(self.ggml_type, "")

    @property
    def k(self) -> int:
        return self.dims[0]

    @property
    def n(self) -> int:
        n = 1
        for d in self.dims[1:]:
            n *= d
        return n


class GgufFile:
    def __init__(self, path: str):
        self._f = open(path, "rb")
        self._m = mmap.mmap(self._f.fileno(), 0, access=mmap.ACCESS_READ)
        self.metadata: Dict[str, object] = {}
        self.tensors: Dict[str, TensorInfo] = {}
        self._parse()

    def close(self) -> None:
        self._m.close()
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # ---- parsing ---------------------------------------------------------------------------------
    def _unpack(self, fmt: str):
        size = struct.calcsize(fmt)
        if self._pos + size > len(self._m):
            raise GpuError("Transfer", "GGUF file is truncated")
        v = struct.unpack_from(fmt, self._m, self._pos)[0]
        self._pos += size
        return v

    def _string(self) -> str:
        n = self._unpack("<Q")
        if self._pos + n > len(self._m):
            raise GpuError("Transfer", "GGUF file is truncated")
        s = bytes(self._m[self._pos:self._pos + n]).decode("utf-8", errors="replace")
        self._pos += n
        return s

    def _value(self, vtype: int):
        if vtype in _SCALAR:
            return self._unpack(_SCALAR[vtype])
        if vtype == 8:
            return self._string()
        if vtype == 9:
            etype, count = self._unpack("<I"), self._unpack("<Q")
            return [self._value(etype) for _ in range(count)]
        raise GpuError("Transfer", f"GGUF metadata value of unknown type {vtype}")

    def _parse(self) -> None:
        self._pos = 0
        if self._unpack("<I") != GGUF_MAGIC:
            raise GpuError("Transfer", "not a GGUF file")
        self.version = self._unpack("<I")
        if self.version not in (2, 3):
            raise GpuError("Transfer", f"GGUF version {self.version} is not supported")
        n_tensors, n_kv = self._unpack("<Q"), self._unpack("<Q")
        for _ in range(n_kv):
            key = self._string()
            self.metadata[key] = self._value(self._unpack("<I"))
        infos = []
        for _ in range(n_tensors):
            name = self._string()
            dims = tuple(self._unpack("<Q") for _ in range(self._unpack("<I")))
            infos.append((name, dims, self._unpack("<I"), self._unpack("<Q")))
        align = int(self.metadata.get("general.alignment", 32))
        data_start = (self._pos + align - 1) // align * align
        for name, dims, gtype, rel in infos:
            count = 1
            for d in dims:
                count *= d
            per, size = _BLOCK.get(gtype, (0, 0))
            nbytes = count // per * size if per and count % per == 0 and (not dims or dims[0] % per == 0) else -1
            if nbytes >= 0 and data_start + rel + nbytes > len(self._m):
                raise GpuError("Transfer", f"GGUF tensor {name} runs past the end of the file")
            self.tensors[name] = TensorInfo(name, dims, gtype, data_start + rel, nbytes)

    # ---- access ---------------------------------------------------------------------------------
    def tensor_bytes(self, name: str) -> np.ndarray:
        """The tensor's bytes as they lie in the file (a view of the mapping)."""
        info = self.tensors[name]
        if info.nbytes < 0:
            raise GpuError("Transfer", f"GGUF tensor {name} has type {info.ggml_type}, which this path does not read")
        return np.frombuffer(self._m, np.uint8, info.nbytes, info.offset)

    def upload(self, ctx: CudaContext, stream: CudaStream, name: str) -> GpuBuffer:
        """The tensor on the GPU, ready for the kernels: uint8 blocks for Q4_K/Q5_K/Q6_K (Q5_K re-packed), float32
        for F32.  Synchronises the stream when a re-pack was needed."""
        info = self.tensors[name]
        raw = self.tensor_bytes(name)
        if info.ggml_type == GGML_F32:
            return GpuBuffer.from_host(ctx, raw.view(np.float32))
        if not info.fmt:
            raise GpuError("Transfer", f"GGUF tensor {name} has type {info.ggml_type}, which this path does not read")
        buf = GpuBuffer.from_host(ctx, raw)
        if info.ggml_type == GGML_Q5_K:
            _check(_lib().trn_q5k_from_ggml(stream.raw() if stream is not None else None, buf.as_ptr(), buf.as_ptr(),
                                            info.nbytes // 176), "KernelLaunch", "q5k_from_ggml")
            stream.synchronize()
        return buf
