"""Seeded synthetic inputs: normal/uniform generators and GGUF block quantizers.

Host-side tooling for tests and benchmarks (``libjoshua_synth.so``, built from
``synth.cpp``).  The block bytes it produces are this build's own; the
reference quantizes only in its tests, through a third-party crate.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libjoshua_synth.so")

Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS, MXFP4 = 8, 10, 12, 14, 16, 39


def build() -> str:
    subprocess.run(["g++", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wextra", "-shared", "-pthread", "-o", _LIB_PATH,
                    os.path.join(_HERE, "synth.cpp")], check=True)
    return _LIB_PATH


_lib = None


def _L() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        u64, sz, f32, vp, i32, u32 = (ctypes.c_uint64, ctypes.c_size_t, ctypes.c_float, ctypes.c_void_p,
                                      ctypes.c_int, ctypes.c_uint32)
        L.jsyn_fill_normal.argtypes = [u64, u64, sz, f32, f32, vp, i32]
        L.jsyn_fill_uniform_u32.argtypes = [u64, u64, sz, u32, vp]
        L.jsyn_quantized_size.argtypes = [u32, sz]
        L.jsyn_quantized_size.restype = sz
        L.jsyn_quantize.argtypes = [u32, vp, sz, vp, i32]
        L.jsyn_normal_quantized.argtypes = [u32, u64, u64, sz, f32, f32, vp, i32]
        _lib = L
    return _lib


def normal(seed: int, shape, sigma: float = 1.0, mean: float = 0.0, start: int = 0, threads: int = 0) -> np.ndarray:
    """f32 N(mean, sigma) array; element i depends only on (seed, start + i)."""
    out = np.empty(shape, dtype=np.float32)
    _L().jsyn_fill_normal(seed, start, out.size, mean, sigma, out.ctypes.data, threads)
    return out


def uniform_u32(seed: int, n: int, bound: int, start: int = 0) -> np.ndarray:
    out = np.empty(n, dtype=np.uint32)
    _L().jsyn_fill_uniform_u32(seed, start, n, bound, out.ctypes.data)
    return out


def quantized_size(qtype: int, n_elems: int) -> int:
    nbytes = _L().jsyn_quantized_size(qtype, n_elems)
    if nbytes == 0 and n_elems:
        raise ValueError(f"type {qtype}: {n_elems} elements is not a whole number of blocks (or unknown type)")
    return nbytes


def quantize(qtype: int, w: np.ndarray, threads: int = 0) -> np.ndarray:
    """Quantize a row-major f32 matrix to packed GGUF blocks (uint8 array)."""
    w = np.ascontiguousarray(w, dtype=np.float32)
    out = np.empty(quantized_size(qtype, w.size), dtype=np.uint8)
    if _L().jsyn_quantize(qtype, w.ctypes.data, w.size, out.ctypes.data, threads) != 0:
        raise ValueError(f"cannot quantize {w.size} elements as type {qtype}")
    return out


def normal_quantized(qtype: int, seed: int, n_elems: int, sigma: float, mean: float = 0.0, start: int = 0,
                     threads: int = 0, out: np.ndarray | None = None) -> np.ndarray:
    """Blocks of quantize(normal(seed, n_elems, sigma)) without the f32 intermediate."""
    nbytes = quantized_size(qtype, n_elems)
    if out is None:
        out = np.empty(nbytes, dtype=np.uint8)
    assert out.dtype == np.uint8 and out.size == nbytes and out.flags.c_contiguous
    if _L().jsyn_normal_quantized(qtype, seed, start, n_elems, mean, sigma, out.ctypes.data, threads) != 0:
        raise ValueError(f"cannot quantize {n_elems} elements as type {qtype}")
    return out
