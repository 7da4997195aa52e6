"""ctypes binding of ``libjoshua_hip.so`` (C ABI in ``include/joshua_hip.h``).

Everything here is plumbing: it passes plain pointers and sizes through the C
ABI exactly as a Rust ``extern "C"`` block would.  There is no CPU fallback: a
missing or unloadable library raises, and so does every failed call.
"""
from __future__ import annotations

import ctypes
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libjoshua_hip.so")

Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS, MXFP4 = 8, 10, 12, 14, 16, 39
ALL_TYPES = (Q8_0, Q2_K, Q4_K, Q6_K, IQ2_XXS, MXFP4)
# formats the reference serves through the canonical decode plus its 8-lane dot
# (reference: src/quant_matmul.rs:228-248; sizes src/gguf_ext.rs:487-500)
Q4_0, Q4_1, Q5_0, Q5_1, Q3_K, Q5_K = 2, 3, 6, 7, 11, 13
GENERIC_TYPES = (Q4_0, Q4_1, Q5_0, Q5_1, Q3_K, Q5_K)
TYPE_NAMES = {Q8_0: "Q8_0", Q2_K: "Q2_K", Q4_K: "Q4_K", Q6_K: "Q6_K", IQ2_XXS: "IQ2_XXS", MXFP4: "MXFP4", Q4_0: "Q4_0",
              Q4_1: "Q4_1", Q5_0: "Q5_0", Q5_1: "Q5_1", Q3_K: "Q3_K", Q5_K: "Q5_K"}

# Every symbol include/joshua_hip.h declares.
EXPORTS = (
    "jq_last_error", "jq_last_kernel", "jq_block_geometry", "jq_init", "jq_upload", "jq_view", "jq_free", "jq_dtype", "jq_rows",
    "jq_cols", "jq_storage_size_in_bytes", "jq_device_ptr", "jq_matmul_t", "jq_matmul_t_f16", "jq_matmul_t_noalloc", "jq_try_matmul_fused", "jq_dequantize", "jq_decode_raw_to_f32", "jq_stream_release",
    "jq_embedding", "jq_stream_synchronize", "jq_moe_create", "jq_moe_free", "jq_moe_route", "jq_moe_forward",
    "jq_mla_create", "jq_mla_free", "jq_mla_forward", "jq_mla_reset", "jq_mla_cached_tokens",
    "jq_qwen3_create", "jq_qwen3_free", "jq_qwen3_set_tensor", "jq_qwen3_forward", "jq_qwen3_greedy", "jq_qwen3_reset",
    "jq_qwen3_get_config", "jq_qwen3_load_gguf", "jq_type_size_bytes", "jq_gguf_open", "jq_gguf_parse", "jq_gguf_close",
    "jq_gguf_version", "jq_gguf_tensor_data_offset", "jq_gguf_tensor_count", "jq_gguf_metadata_count",
    "jq_gguf_tensor_at", "jq_gguf_find_tensor", "jq_gguf_tensor_bytes", "jq_gguf_meta_u32", "jq_gguf_meta_f32",
    "jq_gguf_meta_bool", "jq_gguf_meta_str", "jq_gguf_meta_array_len", "jq_gguf_upload",
    "joshua_npu_init", "joshua_npu_forward", "joshua_npu_reset", "joshua_npu_free",
)


class JoshuaHipError(RuntimeError):
    """A C-ABI call returned nonzero; the message is jq_last_error()."""


class MoeConfig(ctypes.Structure):
    """jq_moe_config of include/joshua_hip.h."""
    _fields_ = [("n_expert", ctypes.c_uint32), ("n_expert_used", ctypes.c_uint32), ("hidden", ctypes.c_uint32),
                ("inter", ctypes.c_uint32), ("gating", ctypes.c_uint32), ("norm_topk", ctypes.c_uint32),
                ("weights_scale", ctypes.c_float), ("n_group", ctypes.c_uint32), ("topk_group", ctypes.c_uint32),
                ("swiglu_clamp", ctypes.c_float), ("swiglu_clamp_shared", ctypes.c_float)]


class MlaConfig(ctypes.Structure):
    """jq_mla_config of include/joshua_hip.h."""
    _fields_ = [("n_embd", ctypes.c_uint32), ("n_head", ctypes.c_uint32), ("q_lora_rank", ctypes.c_uint32),
                ("kv_lora_rank", ctypes.c_uint32), ("qk_nope_head_dim", ctypes.c_uint32),
                ("qk_rope_head_dim", ctypes.c_uint32), ("v_head_dim", ctypes.c_uint32), ("n_ctx", ctypes.c_uint32),
                ("rms_eps", ctypes.c_float), ("rope_theta", ctypes.c_float), ("yarn_factor", ctypes.c_float),
                ("yarn_mscale_all_dim", ctypes.c_float), ("yarn_orig_context_length", ctypes.c_uint32)]


class Qwen3Config(ctypes.Structure):
    """jq_qwen3_config of include/joshua_hip.h."""
    _fields_ = [("n_layer", ctypes.c_uint32), ("hidden", ctypes.c_uint32), ("n_head", ctypes.c_uint32),
                ("n_kv_head", ctypes.c_uint32), ("head_dim", ctypes.c_uint32), ("ffn", ctypes.c_uint32),
                ("vocab", ctypes.c_uint32), ("n_ctx", ctypes.c_uint32), ("rms_eps", ctypes.c_float),
                ("rope_theta", ctypes.c_float), ("n_expert", ctypes.c_uint32), ("n_expert_used", ctypes.c_uint32),
                ("expert_ffn", ctypes.c_uint32), ("norm_topk_prob", ctypes.c_uint32)]


_lib = None


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise JoshuaHipError(
                f"{LIB_PATH} is missing: build it with `python -m joshua_amd.build` (there is no CPU fallback)")
        # One process must hold one HIP runtime.  PyTorch ships its own copy of
        # libamdhip64 under the same soname the library links against, so when
        # torch is installed it is loaded first and the loader binds this
        # library to that copy; without torch the system runtime is used.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = ctypes.CDLL(LIB_PATH)
        sz, u32, vp, i32 = ctypes.c_size_t, ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int
        L.jq_last_error.restype = ctypes.c_char_p
        L.jq_last_kernel.restype = ctypes.c_char_p
        L.jq_block_geometry.argtypes = [u32, ctypes.POINTER(sz), ctypes.POINTER(sz)]
        L.jq_init.argtypes = [i32]
        L.jq_upload.argtypes = [u32, vp, sz, sz, sz, i32, ctypes.POINTER(vp)]
        L.jq_view.argtypes = [vp, sz, sz, sz, ctypes.POINTER(vp)]
        L.jq_free.argtypes = [vp]
        L.jq_free.restype = None
        L.jq_dtype.argtypes = [vp]
        L.jq_dtype.restype = u32
        for f in (L.jq_rows, L.jq_cols, L.jq_storage_size_in_bytes):
            f.argtypes = [vp]
            f.restype = sz
        L.jq_device_ptr.argtypes = [vp]
        L.jq_device_ptr.restype = vp
        L.jq_matmul_t.argtypes = [vp, sz, vp, sz, vp, sz, i32, vp]
        L.jq_matmul_t_f16.argtypes = [vp, sz, vp, sz, vp, sz, i32, vp]
        L.jq_matmul_t_noalloc.argtypes = [vp, sz, vp, sz, vp, sz, vp]
        L.jq_try_matmul_fused.argtypes = [u32, sz, sz, sz, vp, vp, sz, vp, vp]
        L.jq_dequantize.argtypes = [vp, vp, sz, i32, vp]
        L.jq_decode_raw_to_f32.argtypes = [u32, vp, sz, sz, vp, i32, vp]
        L.jq_stream_release.argtypes = [vp]
        L.jq_embedding.argtypes = [vp, vp, sz, vp, sz, i32, vp]
        L.jq_stream_synchronize.argtypes = [vp]
        L.jq_moe_create.argtypes = [ctypes.POINTER(MoeConfig), vp, vp, vp, vp, vp, vp, vp, vp, ctypes.POINTER(vp)]
        L.jq_moe_free.argtypes = [vp]
        L.jq_moe_free.restype = None
        L.jq_moe_route.argtypes = [vp, sz, vp, vp, vp, i32, vp]
        L.jq_moe_forward.argtypes = [vp, sz, vp, vp, i32, vp]
        L.jq_mla_create.argtypes = [ctypes.POINTER(MlaConfig), vp, vp, vp, vp, vp, vp, vp, vp, ctypes.POINTER(vp)]
        L.jq_mla_free.argtypes = [vp]
        L.jq_mla_free.restype = None
        L.jq_mla_forward.argtypes = [vp, sz, sz, vp, vp, i32, vp]
        L.jq_mla_reset.argtypes = [vp]
        L.jq_mla_cached_tokens.argtypes = [vp]
        L.jq_mla_cached_tokens.restype = sz
        L.jq_qwen3_create.argtypes = [ctypes.POINTER(Qwen3Config), ctypes.POINTER(vp)]
        L.jq_qwen3_free.argtypes = [vp]
        L.jq_qwen3_free.restype = None
        L.jq_qwen3_set_tensor.argtypes = [vp, ctypes.c_char_p, u32, vp, sz]
        L.jq_qwen3_forward.argtypes = [vp, vp, u32, u32, vp, i32, vp]
        L.jq_qwen3_greedy.argtypes = [vp, ctypes.POINTER(u32), vp]
        L.jq_qwen3_reset.argtypes = [vp]
        L.jq_qwen3_get_config.argtypes = [vp, ctypes.POINTER(Qwen3Config)]
        L.jq_qwen3_load_gguf.argtypes = [ctypes.c_char_p, u32, ctypes.POINTER(vp)]
        u64 = ctypes.c_uint64
        L.jq_type_size_bytes.argtypes = [u32, sz, ctypes.POINTER(sz)]
        L.jq_gguf_open.argtypes = [ctypes.c_char_p, ctypes.POINTER(vp)]
        L.jq_gguf_parse.argtypes = [vp, sz, ctypes.POINTER(vp)]
        L.jq_gguf_close.argtypes = [vp]
        L.jq_gguf_close.restype = None
        L.jq_gguf_version.argtypes = [vp]
        L.jq_gguf_version.restype = u32
        L.jq_gguf_tensor_data_offset.argtypes = [vp]
        L.jq_gguf_tensor_data_offset.restype = u64
        for f in (L.jq_gguf_tensor_count, L.jq_gguf_metadata_count):
            f.argtypes = [vp]
            f.restype = sz
        L.jq_gguf_tensor_at.argtypes = [vp, sz, ctypes.POINTER(ctypes.c_char_p), ctypes.POINTER(u32), ctypes.POINTER(u32),
                                        ctypes.POINTER(u64), ctypes.POINTER(u64)]
        L.jq_gguf_find_tensor.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(sz)]
        L.jq_gguf_tensor_bytes.argtypes = [vp, sz, ctypes.POINTER(vp), ctypes.POINTER(sz)]
        L.jq_gguf_meta_u32.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(u32)]
        L.jq_gguf_meta_f32.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(ctypes.c_float)]
        L.jq_gguf_meta_bool.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(i32)]
        L.jq_gguf_meta_str.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(vp), ctypes.POINTER(sz)]
        L.jq_gguf_meta_array_len.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(sz)]
        L.jq_gguf_upload.argtypes = [vp, ctypes.c_char_p, ctypes.POINTER(vp)]
        L.joshua_npu_init.argtypes = [ctypes.c_char_p, u32, ctypes.POINTER(u32), ctypes.POINTER(vp)]
        L.joshua_npu_init.restype = ctypes.c_int32
        L.joshua_npu_forward.argtypes = [vp, vp, u32, u32, vp]
        L.joshua_npu_forward.restype = ctypes.c_int32
        L.joshua_npu_reset.argtypes = [vp]
        L.joshua_npu_reset.restype = ctypes.c_int32
        L.joshua_npu_free.argtypes = [vp]
        L.joshua_npu_free.restype = None
        _lib = L
    return _lib


def last_error() -> str:
    return lib().jq_last_error().decode()


def last_kernel() -> str:
    """The kernel the calling thread's last matmul call chose."""
    return lib().jq_last_kernel().decode()


def stream_release(stream: int = 0) -> None:
    """Frees the scratch memory the library keeps for a stream (graphs captured on it become invalid)."""
    _check(lib().jq_stream_release(stream or None))


def decode_raw_to_f32(dtype: int, raw, elems: int):
    """f32 values of raw tensor bytes, or None where the reference's decode_raw_to_f32 answers None
    (src/quant_matmul.rs:36-103); a size mismatch raises with the reference's wording."""
    raw = np.ascontiguousarray(np.frombuffer(raw, dtype=np.uint8) if not isinstance(raw, np.ndarray) else raw.view(np.uint8).reshape(-1))
    out = np.empty(elems, dtype=np.float32)
    rc = lib().jq_decode_raw_to_f32(dtype, raw.ctypes.data if raw.size else None, raw.size, elems,
                                    out.ctypes.data if elems else None, 0, None)
    if rc == 2:
        return None
    _check(rc)
    return out


def _check(rc: int) -> None:
    if rc != 0:
        raise JoshuaHipError(last_error())


def block_geometry(qtype: int) -> tuple[int, int]:
    e, b = ctypes.c_size_t(), ctypes.c_size_t()
    _check(lib().jq_block_geometry(qtype, ctypes.byref(e), ctypes.byref(b)))
    return e.value, b.value


def init(device: int = 0) -> None:
    _check(lib().jq_init(device))


def _host_bytes(blocks) -> np.ndarray:
    a = blocks if isinstance(blocks, np.ndarray) else np.frombuffer(blocks, dtype=np.uint8)
    return np.ascontiguousarray(a.view(np.uint8).reshape(-1))


class Weight:
    """An n x k quantized weight resident in HBM in native block layout: the
    counterpart of the reference's borrowed storage objects
    (reference: src/mmap_tensor.rs:54-60,127-203)."""

    def __init__(self, handle: int, parent: "Weight | None" = None):
        self._h = ctypes.c_void_p(handle)
        self._parent = parent  # keeps the aliased allocation alive

    @classmethod
    def upload(cls, qtype: int, blocks, n: int, k: int) -> "Weight":
        raw = _host_bytes(blocks)
        out = ctypes.c_void_p()
        _check(lib().jq_upload(qtype, raw.ctypes.data, raw.size, n, k, 0, ctypes.byref(out)))
        return cls(out.value)

    @classmethod
    def upload_device(cls, qtype: int, dev_ptr: int, nbytes: int, n: int, k: int) -> "Weight":
        out = ctypes.c_void_p()
        _check(lib().jq_upload(qtype, dev_ptr, nbytes, n, k, 1, ctypes.byref(out)))
        return cls(out.value)

    def view(self, byte_offset: int, n: int, k: int) -> "Weight":
        out = ctypes.c_void_p()
        _check(lib().jq_view(self._h, byte_offset, n, k, ctypes.byref(out)))
        return Weight(out.value, parent=self)

    def close(self) -> None:
        if self._h:
            lib().jq_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def handle(self) -> ctypes.c_void_p:
        return self._h

    @property
    def dtype(self) -> int:
        return lib().jq_dtype(self._h)

    @property
    def n(self) -> int:
        return lib().jq_rows(self._h)

    @property
    def k(self) -> int:
        return lib().jq_cols(self._h)

    @property
    def nbytes(self) -> int:
        return lib().jq_storage_size_in_bytes(self._h)

    @property
    def device_ptr(self) -> int:
        return lib().jq_device_ptr(self._h)

    # -- host-pointer calls (numpy in, numpy out) --------------------------------
    def matmul_t(self, m: int, lhs: np.ndarray, dst: np.ndarray | None = None) -> np.ndarray:
        x = np.ascontiguousarray(np.asarray(lhs, dtype=np.float32).reshape(-1))
        if dst is None:
            dst = np.empty(m * self.n, dtype=np.float32)
        assert dst.dtype == np.float32 and dst.flags.c_contiguous
        _check(lib().jq_matmul_t(self._h, m, x.ctypes.data, x.size, dst.ctypes.data, dst.size, 0, None))
        return dst.reshape(m, self.n) if dst.size == m * self.n else dst

    def matmul_t_f16(self, m: int, lhs: np.ndarray) -> np.ndarray:
        """f16 activations in, f16 results out (reference: src/mmap_tensor.rs:136-138 matmul_t_f16)."""
        x = np.ascontiguousarray(np.asarray(lhs, dtype=np.float16).reshape(-1))
        dst = np.empty(m * self.n, dtype=np.float16)
        _check(lib().jq_matmul_t_f16(self._h, m, x.ctypes.data, x.size, dst.ctypes.data, dst.size, 0, None))
        return dst.reshape(m, self.n)

    def dequantize(self) -> np.ndarray:
        out = np.empty(self.n * self.k, dtype=np.float32)
        _check(lib().jq_dequantize(self._h, out.ctypes.data, out.size, 0, None))
        return out.reshape(self.n, self.k)

    def embedding(self, ids) -> np.ndarray:
        ids = np.ascontiguousarray(ids, dtype=np.uint32)
        out = np.empty(ids.size * self.k, dtype=np.float32)
        _check(lib().jq_embedding(self._h, ids.ctypes.data, ids.size, out.ctypes.data, out.size, 0, None))
        return out.reshape(ids.size, self.k)

    # -- device-pointer calls (raw addresses; inputs already in HBM) -------------
    def matmul_t_dev(self, m: int, lhs_ptr: int, lhs_len: int, dst_ptr: int, dst_len: int, stream: int = 0) -> None:
        _check(lib().jq_matmul_t(self._h, m, lhs_ptr, lhs_len, dst_ptr, dst_len, 1, stream or None))

    def matmul_t_f16_dev(self, m: int, lhs_ptr: int, lhs_len: int, dst_ptr: int, dst_len: int, stream: int = 0) -> None:
        _check(lib().jq_matmul_t_f16(self._h, m, lhs_ptr, lhs_len, dst_ptr, dst_len, 1, stream or None))

    def matmul_t_noalloc(self, m: int, lhs_ptr: int, lhs_len: int, dst_ptr: int, dst_len: int, stream: int = 0) -> None:
        """The same product through the entry point that allocates no device memory."""
        _check(lib().jq_matmul_t_noalloc(self._h, m, lhs_ptr, lhs_len, dst_ptr, dst_len, stream or None))


def try_matmul_fused(qtype: int, mkn, lhs_ptr: int, blocks_ptr: int, nbytes: int, dst_ptr: int, stream: int = 0) -> bool:
    """True when a kernel ran; False when the call declined (dst untouched), as
    the reference's free function does (src/kquant_dot.rs:120-133)."""
    m, k, n = mkn
    return lib().jq_try_matmul_fused(qtype, m, k, n, lhs_ptr, blocks_ptr, nbytes, dst_ptr, stream or None) == 0


def stream_synchronize(stream: int = 0) -> None:
    _check(lib().jq_stream_synchronize(stream or None))


class Moe:
    """A mixture-of-experts layer on the device (reference: src/quantized_qwen3_moe.rs:404-520,
    src/quantized_deepseek2.rs:508-672)."""

    def __init__(self, cfg: MoeConfig, router_w: np.ndarray, gate_exps: Weight, up_exps: Weight, down_exps: Weight,
                 router_bias: np.ndarray | None = None, shared: "tuple[Weight, Weight, Weight] | None" = None):
        self.cfg = cfg
        self._keep = (gate_exps, up_exps, down_exps, shared)
        rw = np.ascontiguousarray(router_w, dtype=np.float32)
        assert rw.shape == (cfg.n_expert, cfg.hidden)
        rb = None if router_bias is None else np.ascontiguousarray(router_bias, dtype=np.float32)
        sh = [w.handle for w in shared] if shared else [None, None, None]
        out = ctypes.c_void_p()
        _check(lib().jq_moe_create(ctypes.byref(cfg), rw.ctypes.data, None if rb is None else rb.ctypes.data,
                                   gate_exps.handle, up_exps.handle, down_exps.handle, sh[0], sh[1], sh[2],
                                   ctypes.byref(out)))
        self._h = out

    def close(self) -> None:
        if self._h:
            lib().jq_moe_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def route(self, x: np.ndarray):
        x = np.ascontiguousarray(x, dtype=np.float32)
        t = x.shape[0]
        ids = np.empty((t, self.cfg.n_expert_used), np.uint32)
        w = np.empty((t, self.cfg.n_expert_used), np.float32)
        _check(lib().jq_moe_route(self._h, t, x.ctypes.data, ids.ctypes.data, w.ctypes.data, 0, None))
        return ids, w

    def forward(self, x: np.ndarray) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        y = np.empty_like(x)
        _check(lib().jq_moe_forward(self._h, x.shape[0], x.ctypes.data, y.ctypes.data, 0, None))
        return y

    def forward_dev(self, n_tokens: int, x_ptr: int, y_ptr: int, stream: int = 0) -> None:
        _check(lib().jq_moe_forward(self._h, n_tokens, x_ptr, y_ptr, 1, stream or None))


class Mla:
    """The multi-head latent attention block of the reference's deepseek2 graph on the device
    (reference: src/quantized_deepseek2.rs:374-503 Attention).  `q` is attn_q, or with a low-rank Q
    projection the triple (attn_q_a, attn_q_a_norm, attn_q_b); `kv_b` is a Weight or a dense f32
    [n_head * (qk_nope + v_head_dim), kv_lora_rank] array."""

    def __init__(self, cfg: MlaConfig, q, kv_a_mqa: Weight, kv_a_norm: np.ndarray, kv_b, o_proj: Weight):
        self.cfg = cfg
        q_a, q_norm, q_b = q if isinstance(q, tuple) else (q, None, None)
        qn = None if q_norm is None else np.ascontiguousarray(q_norm, dtype=np.float32)
        kn = np.ascontiguousarray(kv_a_norm, dtype=np.float32)
        dense = None if isinstance(kv_b, Weight) else np.ascontiguousarray(kv_b, dtype=np.float32)
        if dense is not None:
            assert dense.size == cfg.n_head * (cfg.qk_nope_head_dim + cfg.v_head_dim) * cfg.kv_lora_rank
        assert kn.size == cfg.kv_lora_rank and (qn is None or qn.size == cfg.q_lora_rank)
        self._keep = (q_a, q_b, kv_a_mqa, kv_b, o_proj)
        out = ctypes.c_void_p()
        _check(lib().jq_mla_create(ctypes.byref(cfg), q_a.handle, None if qn is None else qn.ctypes.data,
                                   None if q_b is None else q_b.handle, kv_a_mqa.handle, kn.ctypes.data,
                                   kv_b.handle if dense is None else None, None if dense is None else dense.ctypes.data,
                                   o_proj.handle, ctypes.byref(out)))
        self._h = out

    def close(self) -> None:
        if self._h:
            lib().jq_mla_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def forward(self, x: np.ndarray, pos: int) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        y = np.empty_like(x)
        _check(lib().jq_mla_forward(self._h, x.shape[0], pos, x.ctypes.data, y.ctypes.data, 0, None))
        return y

    def forward_dev(self, n_tokens: int, pos: int, x_ptr: int, y_ptr: int, stream: int = 0) -> None:
        _check(lib().jq_mla_forward(self._h, n_tokens, pos, x_ptr, y_ptr, 1, stream or None))

    def reset(self) -> None:
        _check(lib().jq_mla_reset(self._h))

    @property
    def cached_tokens(self) -> int:
        return int(lib().jq_mla_cached_tokens(self._h))


class Qwen3:
    """The dense Qwen3 decoder graph on the device, fed and stepped like the reference's
    model object (reference: src/quantized_qwen3_moe.rs:792-826 forward / clear_kv_cache;
    driver loop src/engine.rs:1149-1294)."""

    def __init__(self, cfg: Qwen3Config):
        self.cfg = cfg
        out = ctypes.c_void_p()
        _check(lib().jq_qwen3_create(ctypes.byref(cfg), ctypes.byref(out)))
        self._h = out

    @classmethod
    def from_gguf(cls, path: str, n_ctx: int = 0) -> "Qwen3":
        """Loads a dense qwen3 GGUF file: configuration from its metadata, every tensor
        uploaded once in native layout (reference: src/quantized_qwen3_moe.rs:90-147,725-775)."""
        out = ctypes.c_void_p()
        _check(lib().jq_qwen3_load_gguf(os.fsencode(path), n_ctx, ctypes.byref(out)))
        self = cls.__new__(cls)
        self._h = out
        self.cfg = Qwen3Config()
        _check(lib().jq_qwen3_get_config(out, ctypes.byref(self.cfg)))
        return self

    def close(self) -> None:
        if self._h:
            lib().jq_qwen3_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def set_tensor(self, name: str, qtype: int, data) -> None:
        """qtype 0: f32 vector; else packed blocks of that GGUF type."""
        a = np.ascontiguousarray(data, dtype=np.float32) if qtype == 0 else _host_bytes(data)
        _check(lib().jq_qwen3_set_tensor(self._h, name.encode(), qtype, a.ctypes.data, a.nbytes))

    def forward(self, tokens, pos: int) -> np.ndarray:
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.empty(self.cfg.vocab, np.float32)
        _check(lib().jq_qwen3_forward(self._h, t.ctypes.data, t.size, pos, logits.ctypes.data, 0, None))
        return logits

    def forward_only(self, tokens, pos: int, stream: int = 0) -> None:
        """Enqueues the step and leaves the logits on the device (for greedy())."""
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        _check(lib().jq_qwen3_forward(self._h, t.ctypes.data, t.size, pos, None, 1, stream or None))

    def greedy(self, stream: int = 0) -> int:
        tok = ctypes.c_uint32()
        _check(lib().jq_qwen3_greedy(self._h, ctypes.byref(tok), stream or None))
        return tok.value

    def reset(self) -> None:
        _check(lib().jq_qwen3_reset(self._h))


def type_size_bytes(qtype: int, elems: int) -> "int | None":
    """Bytes of `elems` elements of a raw GGUF type id, or None
    (reference: src/gguf_ext.rs:483-512)."""
    out = ctypes.c_size_t()
    return out.value if lib().jq_type_size_bytes(qtype, elems, ctypes.byref(out)) == 0 else None


class Gguf:
    """A GGUF file mapped read-only, or a header parsed from bytes: the tensor directory with
    raw type ids, metadata scalars, and uploads straight from the mapping
    (reference: src/gguf_ext.rs:117-146 RawTensorInfo / GgufHeader, :400-480 read_header)."""

    def __init__(self, handle: ctypes.c_void_p):
        self._h = handle

    @classmethod
    def open(cls, path: str) -> "Gguf":
        out = ctypes.c_void_p()
        _check(lib().jq_gguf_open(os.fsencode(path), ctypes.byref(out)))
        return cls(out)

    @classmethod
    def parse(cls, data: bytes) -> "Gguf":
        out = ctypes.c_void_p()
        buf = (ctypes.c_char * max(len(data), 1)).from_buffer_copy(data or b"\0")
        _check(lib().jq_gguf_parse(ctypes.addressof(buf), len(data), ctypes.byref(out)))
        return cls(out)

    def close(self) -> None:
        if self._h:
            lib().jq_gguf_close(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self) -> int:
        return lib().jq_gguf_version(self._h)

    @property
    def tensor_data_offset(self) -> int:
        return lib().jq_gguf_tensor_data_offset(self._h)

    @property
    def metadata_count(self) -> int:
        return lib().jq_gguf_metadata_count(self._h)

    def tensors(self) -> dict:
        """name -> (raw type id, dims in row-major order, offset from tensor_data_offset)."""
        out = {}
        for i in range(lib().jq_gguf_tensor_count(self._h)):
            name, ty, nd, off = ctypes.c_char_p(), ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint64()
            dims = (ctypes.c_uint64 * 8)()
            _check(lib().jq_gguf_tensor_at(self._h, i, ctypes.byref(name), ctypes.byref(ty), ctypes.byref(nd), dims,
                                           ctypes.byref(off)))
            out[name.value.decode(errors="replace")] = (ty.value, list(dims[:nd.value]), off.value)
        return out

    def tensor_bytes(self, name: str) -> np.ndarray:
        """A copy of the tensor's bytes out of the mapping."""
        idx, p, n = ctypes.c_size_t(), ctypes.c_void_p(), ctypes.c_size_t()
        _check(lib().jq_gguf_find_tensor(self._h, name.encode(), ctypes.byref(idx)))
        _check(lib().jq_gguf_tensor_bytes(self._h, idx.value, ctypes.byref(p), ctypes.byref(n)))
        return np.frombuffer(ctypes.string_at(p.value, n.value), dtype=np.uint8).copy()

    def meta_u32(self, key: str) -> "int | None":
        v = ctypes.c_uint32()
        return v.value if lib().jq_gguf_meta_u32(self._h, key.encode(), ctypes.byref(v)) == 0 else None

    def meta_f32(self, key: str) -> "float | None":
        v = ctypes.c_float()
        return v.value if lib().jq_gguf_meta_f32(self._h, key.encode(), ctypes.byref(v)) == 0 else None

    def meta_bool(self, key: str) -> "bool | None":
        v = ctypes.c_int()
        return bool(v.value) if lib().jq_gguf_meta_bool(self._h, key.encode(), ctypes.byref(v)) == 0 else None

    def meta_str(self, key: str) -> "bytes | None":
        """The string's bytes with trailing NULs dropped (decode with errors="replace" for text)."""
        p, n = ctypes.c_void_p(), ctypes.c_size_t()
        if lib().jq_gguf_meta_str(self._h, key.encode(), ctypes.byref(p), ctypes.byref(n)) != 0:
            return None
        return ctypes.string_at(p.value, n.value)

    def meta_array_len(self, key: str) -> "int | None":
        n = ctypes.c_size_t()
        return n.value if lib().jq_gguf_meta_array_len(self._h, key.encode(), ctypes.byref(n)) == 0 else None

    def upload(self, name: str) -> Weight:
        out = ctypes.c_void_p()
        _check(lib().jq_gguf_upload(self._h, name.encode(), ctypes.byref(out)))
        return Weight(out.value)


class NpuPlugin:
    """The library driven through the four joshua_npu_* symbols, the way the reference engine
    drives a backend plugin (reference: src/npu/vendor.rs:95-121 init, :150-185 forward_into,
    :244-251 free on drop).  Failures surface as the plugin's return codes."""

    def __init__(self, model_path: str, n_ctx: int):
        vocab, h = ctypes.c_uint32(), ctypes.c_void_p()
        self.rc = lib().joshua_npu_init(os.fsencode(model_path), n_ctx, ctypes.byref(vocab), ctypes.byref(h))
        self.vocab, self._h = vocab.value, h

    def forward(self, tokens, pos: int) -> "tuple[int, np.ndarray]":
        t = np.ascontiguousarray(tokens, dtype=np.uint32)
        logits = np.zeros(self.vocab, np.float32)
        rc = lib().joshua_npu_forward(self._h, t.ctypes.data, t.size, pos, logits.ctypes.data)
        return rc, logits

    def reset(self) -> int:
        return lib().joshua_npu_reset(self._h)

    def close(self) -> None:
        if self._h:
            lib().joshua_npu_free(self._h)
            self._h = ctypes.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
