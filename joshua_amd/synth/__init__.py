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


# (block elements, block bytes, [(byte offset of an f16 scale, its magnitude)]) of the formats that have no
# quantizer here: every byte pattern is a valid block, so seeded random bytes with sane scales stand in
# for quantized weights of roughly N(0, 0.02).
_RANDOM_LAYOUT = {
    2: (32, 18, [(0, 2.0 ** -8)]), 3: (32, 20, [(0, 2.0 ** -8), (2, -7.5 * 2.0 ** -8)]),
    6: (32, 22, [(0, 2.0 ** -9)]), 7: (32, 24, [(0, 2.0 ** -9), (2, -15.5 * 2.0 ** -9)]),
    11: (256, 110, [(108, 2.0 ** -12)]), 13: (256, 176, [(0, 2.0 ** -14), (2, 2.0 ** -13)]),
}


def random_blocks(qtype: int, seed: int, n_elems: int) -> np.ndarray:
    """Packed blocks of Q4_0, Q4_1, Q5_0, Q5_1, Q3_K or Q5_K (ids 2, 3, 6, 7, 11, 13) holding seeded random
    quants and scales within a factor of two of a per-format magnitude (negative for the offsets of Q4_1
    and Q5_1, which centres their weights)."""
    elems, nbytes, scales = _RANDOM_LAYOUT[qtype]
    if n_elems % elems:
        raise ValueError(f"type {qtype}: {n_elems} elements is not a whole number of blocks")
    rng = np.random.default_rng(seed * 1000 + qtype)
    blk = rng.integers(0, 256, size=(n_elems // elems, nbytes), dtype=np.uint8)
    for off, mag in scales:
        v = mag * rng.uniform(0.5, 1.0, size=blk.shape[0])
        blk[:, off:off + 2] = v.astype(np.float16).view(np.uint8).reshape(-1, 2)
    return blk.reshape(-1)
