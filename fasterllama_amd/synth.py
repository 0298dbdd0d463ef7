"""Seeded synthetic inputs (host side), shared by the tests and the benchmark.

Backed by fasterllama_amd/lib/libfl_synth.so (csrc/fl_synth.c): counter-based splitmix64 +
Box-Muller, so a tensor element depends only on (seed, tensor id, index).
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libfl_synth.so")

TENSOR_Q, TENSOR_K_NEW, TENSOR_V_NEW, TENSOR_K_CACHE, TENSOR_V_CACHE, TENSOR_LENS = 1, 2, 3, 4, 5, 6
DEFAULT_SEED = 1234

_lib = None


def _load() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: run `python -m fasterllama_amd.build synth`")
        lib = C.CDLL(LIB_PATH)
        for name in ("fl_synth_normal_f32", "fl_synth_normal_f16"):
            fn = getattr(lib, name)
            fn.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_float, C.c_int]
            fn.restype = None
        lib.fl_synth_uniform_i32.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int32, C.c_int32]
        lib.fl_synth_uniform_i32.restype = None
        lib.fl_synth_u64.argtypes = [C.c_uint64, C.c_uint64, C.c_uint64]
        lib.fl_synth_u64.restype = C.c_uint64
        _lib = lib
    return _lib


def host_threads() -> int:
    return max(1, min(16, os.cpu_count() or 1))


def normal(shape, dtype, tensor_id: int, seed: int = DEFAULT_SEED, scale: float = 1.0,
           index0: int = 0, out: np.ndarray | None = None) -> np.ndarray:
    """N(0,1)*scale tensor of `shape`; dtype np.float32 or np.float16 (rounded nearest-even)."""
    dtype = np.dtype(dtype)
    arr = out if out is not None else np.empty(shape, dtype=dtype)
    assert arr.flags.c_contiguous and arr.dtype == dtype
    fn = {np.dtype(np.float32): "fl_synth_normal_f32", np.dtype(np.float16): "fl_synth_normal_f16"}[dtype]
    getattr(_load(), fn)(arr.ctypes.data, arr.size, seed, tensor_id, index0, scale, host_threads())
    return arr


def uniform_int(n: int, lo: int, hi: int, tensor_id: int = TENSOR_LENS, seed: int = DEFAULT_SEED) -> np.ndarray:
    """n integers uniform in [lo, hi] (inclusive)."""
    arr = np.empty(n, dtype=np.int32)
    _load().fl_synth_uniform_i32(arr.ctypes.data, n, seed, tensor_id, lo, hi)
    return arr


def freq_cis_table(rows: int, size_per_head: int, base: float = 10000.0) -> np.ndarray:
    """Host RoPE table [rows, D]: row r = [cos(r w_0), sin(r w_0), cos(r w_1), ...], w_i = base^(-2i/D),
    evaluated in float64 and rounded once (layout of decoding_kernels.cu:100-114)."""
    i = np.arange(size_per_head // 2, dtype=np.float64)
    w = np.power(np.float64(base), -2.0 * i / size_per_head)
    theta = np.arange(rows, dtype=np.float64)[:, None] * w[None, :]
    t = np.empty((rows, size_per_head), dtype=np.float32)
    t[:, 0::2] = np.cos(theta)
    t[:, 1::2] = np.sin(theta)
    return t
