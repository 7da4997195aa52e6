"""ctypes front end of the CPU oracle (``oracle/liboracle.so``).

TEST INFRASTRUCTURE, NOT PRODUCT CODE: only ``tests/``, the smoke check and
the benchmark's CPU-baseline leg import this package.  The library restates the
reference's x86_64 quantized-matmul path (reference: src/kquant_dot.rs,
src/quant_matmul.rs, src/iq2xxs.rs, src/mxfp4.rs, src/simd.rs); pin status per
function is listed in ``joshua_oracle.h``.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS, MXFP4 = 8, 10, 12, 14, 16, 39
ALL_TYPES = (Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS, MXFP4)
Q4_0, Q4_1, Q5_0, Q5_1, Q3_K, Q5_K = 2, 3, 6, 7, 11, 13
GENERIC_TYPES = (Q4_0, Q4_1, Q5_0, Q5_1, Q3_K, Q5_K)   # decoded by to_float, multiplied by the 8-lane dot
TYPE_NAMES = {Q8_0: "Q8_0", Q2_K: "Q2_K", Q4_K: "Q4_K", Q6_K: "Q6_K", IQ2_XXS: "IQ2_XXS", MXFP4: "MXFP4", 2: "Q4_0",
              3: "Q4_1", 6: "Q5_0", 7: "Q5_1", 11: "Q3_K", 13: "Q5_K"}


def build(force: bool = False) -> str:
    """Compile the oracle with its Makefile; returns the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-s", "-C", _HERE], check=True)
    return _LIB_PATH


class OracleError(RuntimeError):
    pass


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        sz, u32, vp, fp = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_void_p
        L.orc_block_geometry.argtypes = [u32, ctypes.POINTER(sz), ctypes.POINTER(sz)]
        L.orc_dequantize.argtypes = [u32, vp, sz, fp]
        L.orc_decode_raw_to_f32.argtypes = [u32, vp, sz, sz, fp]
        L.orc_matmul_t.argtypes = [u32, sz, sz, sz, fp, sz, vp, sz, fp, sz]
        L.orc_matmul_t_avx2.argtypes = [u32, sz, sz, sz, fp, sz, vp, sz, fp, sz, ctypes.c_int]
        L.orc_iq2xxs_matmul_scalar.argtypes = [sz, sz, sz, fp, sz, vp, sz, fp, sz]
        L.orc_last_error.restype = ctypes.c_char_p
        L.orc_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.orc_f16_to_f32.restype = ctypes.c_float
        L.orc_e8m0.argtypes = [ctypes.c_uint8, ctypes.POINTER(ctypes.c_int)]
        L.orc_e8m0.restype = ctypes.c_float
        L.orc_iq2xxs_grid.argtypes = [ctypes.c_int, ctypes.c_void_p]
        L.orc_iq2xxs_signs.argtypes = [ctypes.c_uint]
        L.orc_iq2xxs_signs.restype = ctypes.c_uint8
        _lib = L
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        raise OracleError(lib().orc_last_error().decode())


def block_geometry(qtype: int) -> tuple[int, int]:
    """(elements, bytes) per block."""
    e, b = ctypes.c_size_t(), ctypes.c_size_t()
    if lib().orc_block_geometry(qtype, ctypes.byref(e), ctypes.byref(b)) != 0:
        raise OracleError(f"unknown tensor type {qtype}")
    return e.value, b.value


def _bytes_arr(blocks) -> np.ndarray:
    a = np.frombuffer(blocks, dtype=np.uint8) if not isinstance(blocks, np.ndarray) else blocks
    return np.ascontiguousarray(a.view(np.uint8).reshape(-1))


def dequantize(qtype: int, blocks) -> np.ndarray:
    """Canonical decode of whole blocks to f32."""
    raw = _bytes_arr(blocks)
    elems, nbytes = block_geometry(qtype)
    if raw.size % nbytes:
        raise OracleError(f"{raw.size} bytes is not a whole number of {nbytes} byte blocks")
    nblocks = raw.size // nbytes
    out = np.empty(nblocks * elems, dtype=np.float32)
    _check(lib().orc_dequantize(qtype, raw.ctypes.data, nblocks, out.ctypes.data))
    return out


def decode_raw_to_f32(dtype: int, raw, elems: int):
    """The reference's decode_raw_to_f32 (src/quant_matmul.rs:36-103): f32 values, or None where the reference
    answers None (F32 and types without a decoder there)."""
    raw = _bytes_arr(raw)
    out = np.empty(elems, dtype=np.float32)
    rc = lib().orc_decode_raw_to_f32(dtype, raw.ctypes.data, raw.size, elems, out.ctypes.data)
    if rc == 2:
        return None
    _check(rc)
    return out


def matmul_t(qtype: int, mkn, lhs, blocks, *, avx2: bool = False, threads: int = 0, dst=None) -> np.ndarray:
    """dst[m,n] = lhs[m,k] . W[n,k]^T in the reference's operation order.

    ``lhs`` is used at its own length (not reshaped) so the shape checks of the
    reference can be exercised; ``dst`` may be passed to test assign semantics.
    """
    m, k, n = mkn
    x = np.ascontiguousarray(np.asarray(lhs, dtype=np.float32).reshape(-1))
    raw = _bytes_arr(blocks)
    if dst is None:
        dst = np.empty(m * n, dtype=np.float32)
    assert dst.dtype == np.float32 and dst.flags.c_contiguous
    if avx2:
        rc = lib().orc_matmul_t_avx2(qtype, m, k, n, x.ctypes.data, x.size, raw.ctypes.data, raw.size,
                                     dst.ctypes.data, dst.size, threads)
    else:
        rc = lib().orc_matmul_t(qtype, m, k, n, x.ctypes.data, x.size, raw.ctypes.data, raw.size,
                                dst.ctypes.data, dst.size)
    _check(rc)
    return dst.reshape(m, n) if dst.size == m * n else dst


def matmul_t_f16(qtype: int, mkn, lhs, blocks, *, avx2: bool = False) -> np.ndarray:
    """f16 activations in, f16 results out: widen to f32 (exact), the f32 product, round to f16 (nearest even,
    overflow to infinity), as the reference's wrappers do (src/mxfp4.rs:242-258, src/iq2xxs.rs:396-412;
    the k-quant types go through candle's matmul_f16, src/mmap_tensor.rs:136-138, whose f16 result is the
    same rounding of an f32 sum)."""
    m, k, n = mkn
    x16 = np.asarray(lhs, dtype=np.float16)
    return matmul_t(qtype, mkn, x16.astype(np.float32), blocks, avx2=avx2).astype(np.float16)


def iq2xxs_matmul_scalar(mkn, lhs, blocks) -> np.ndarray:
    m, k, n = mkn
    x = np.ascontiguousarray(np.asarray(lhs, dtype=np.float32).reshape(-1))
    raw = _bytes_arr(blocks)
    dst = np.full(m * n, 77.0, dtype=np.float32)
    _check(lib().orc_iq2xxs_matmul_scalar(m, k, n, x.ctypes.data, x.size, raw.ctypes.data, raw.size,
                                          dst.ctypes.data, dst.size))
    return dst.reshape(m, n)


def f16_to_f32(h: int) -> float:
    return float(lib().orc_f16_to_f32(h))


def e8m0(e: int):
    ok = ctypes.c_int()
    v = lib().orc_e8m0(e, ctypes.byref(ok))
    return float(v) if ok.value else None


def iq2xxs_grid_table() -> np.ndarray:
    """The expanded 256x8 codebook."""
    out = np.empty((256, 8), dtype=np.uint8)
    for i in range(256):
        lib().orc_iq2xxs_grid(i, out[i].ctypes.data)
    return out


def have_avx2() -> bool:
    return bool(lib().orc_have_avx2())


def default_threads() -> int:
    return int(lib().orc_default_threads())
