"""ctypes loader for the C oracle (oracle/kquant_ref.c) and the CPU baseline
(oracle/cpu_baseline.cpp).  Test/bench infrastructure only."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
FMT = {"q4k": 4, "q5k": 5, "q6k": 6}
SB = {"q4k": 144, "q5k": 176, "q6k": 210}


def build() -> None:
    subprocess.run(["make", "-C", _HERE, "-s", "-B", "all"], check=True)


def _load(name: str) -> C.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        subprocess.run(["make", "-C", _HERE, "-s", "all"], check=True)
    return C.CDLL(path)


_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)


def _p(a: np.ndarray, t):
    return a.ctypes.data_as(t)


class COracle:
    def __init__(self) -> None:
        L = self.lib = _load("libkquant_oracle.so")
        L.kq_dequant.argtypes = [C.c_int, C.c_int, _u8p, C.c_size_t, _f32p]
        L.kq_dequant.restype = None
        L.kq_gemv_fp64.argtypes = [C.c_int, C.c_int, _u8p, _f32p, C.c_uint32, C.c_uint32, _f64p]
        L.kq_gemv_fp64.restype = None
        L.kq_gemv_ref_order_f32.argtypes = [C.c_int, _u8p, _f32p, C.c_uint32, C.c_uint32, _f32p]
        L.kq_gemv_ref_order_f32.restype = None
        L.kq_gemm_fp64.argtypes = [C.c_int, C.c_int, _u8p, _f32p, C.c_uint32, C.c_uint32, C.c_uint32, _f64p]
        L.kq_gemm_fp64.restype = None
        L.kq_dequant_simplified.argtypes = [_u8p, C.c_size_t, _f32p]
        L.kq_dequant_simplified.restype = None
        L.kq_gemm_simplified_fp64.argtypes = [_u8p, _f32p, C.c_uint32, C.c_uint32, C.c_uint32, _f64p]
        L.kq_gemm_simplified_fp64.restype = None

    def dequant_simplified(self, buf: np.ndarray) -> np.ndarray:
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        n_blocks = buf.size // 18
        out = np.empty((n_blocks, 32), np.float32)
        self.lib.kq_dequant_simplified(_p(buf, _u8p), n_blocks, _p(out, _f32p))
        return out

    def gemm_simplified_fp64(self, buf, a, m: int, n: int, k: int) -> np.ndarray:
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        a = np.ascontiguousarray(a, np.float32)
        c = np.empty((m, n), np.float64)
        self.lib.kq_gemm_simplified_fp64(_p(buf, _u8p), _p(a, _f32p), m, n, k, _p(c, _f64p))
        return c

    def dequant(self, fmt: str, buf: np.ndarray, policy: int = 0) -> np.ndarray:
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        n_sb = buf.size // SB[fmt]
        out = np.empty((n_sb, 256), np.float32)
        self.lib.kq_dequant(FMT[fmt], policy, _p(buf, _u8p), n_sb, _p(out, _f32p))
        return out

    def gemv_fp64(self, fmt: str, buf, x, k: int, n: int, policy: int = 0) -> np.ndarray:
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(n, np.float64)
        self.lib.kq_gemv_fp64(FMT[fmt], policy, _p(buf, _u8p), _p(x, _f32p), k, n, _p(y, _f64p))
        return y

    def gemv_ref_order_f32(self, fmt: str, buf, x, k: int, n: int) -> np.ndarray:
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(n, np.float32)
        self.lib.kq_gemv_ref_order_f32(FMT[fmt], _p(buf, _u8p), _p(x, _f32p), k, n, _p(y, _f32p))
        return y

    def gemm_fp64(self, fmt: str, buf, a, m: int, n: int, k: int, policy: int = 0) -> np.ndarray:
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        a = np.ascontiguousarray(a, np.float32)
        c = np.empty((m, n), np.float64)
        self.lib.kq_gemm_fp64(FMT[fmt], policy, _p(buf, _u8p), _p(a, _f32p), m, n, k, _p(c, _f64p))
        return c


class CpuBaseline:
    def __init__(self) -> None:
        L = self.lib = _load("libkquant_cpu_baseline.so")
        L.kq_cpu_threads.restype = C.c_int
        L.kq_cpu_has_avx2.restype = C.c_int
        L.kq_cpu_decode_block.argtypes = [C.c_int, _u8p, _f32p]
        L.kq_cpu_decode_block.restype = None
        L.kq_cpu_dequant_matvec.argtypes = [C.c_int, _u8p, _f32p, C.c_uint32, C.c_uint32, _f32p, C.c_int, C.c_int]
        L.kq_cpu_dequant_matvec.restype = C.c_double
        L.kq_cpu_matvec_f32.argtypes = [_f32p, _f32p, C.c_uint32, C.c_uint32, _f32p, C.c_int, C.c_int]
        L.kq_cpu_matvec_f32.restype = C.c_double

    def threads(self) -> int:
        return int(self.lib.kq_cpu_threads())

    def has_avx2(self) -> bool:
        return bool(self.lib.kq_cpu_has_avx2())

    def decode_block(self, fmt: str, block: np.ndarray) -> np.ndarray:
        block = np.ascontiguousarray(block, np.uint8).reshape(-1)
        out = np.empty(256, np.float32)
        self.lib.kq_cpu_decode_block(FMT[fmt], _p(block, _u8p), _p(out, _f32p))
        return out

    def dequant_matvec(self, fmt: str, buf, x, k: int, n: int, threads: int, reps: int = 1):
        buf = np.ascontiguousarray(buf, np.uint8).reshape(-1)
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(n, np.float32)
        sec = self.lib.kq_cpu_dequant_matvec(FMT[fmt], _p(buf, _u8p), _p(x, _f32p), k, n, _p(y, _f32p), threads, reps)
        return y, float(sec)

    def matvec_f32(self, w: np.ndarray, x, threads: int, reps: int = 1):
        w = np.ascontiguousarray(w, np.float32)
        n, k = w.shape
        x = np.ascontiguousarray(x, np.float32)
        y = np.empty(n, np.float32)
        sec = self.lib.kq_cpu_matvec_f32(_p(w, _f32p), _p(x, _f32p), k, n, _p(y, _f32p), threads, reps)
        return y, float(sec)
