"""MI355X-native quantized matmul for GGUF blocks (drop-in for joshua's
``matmul_t`` hot path).  The compute lives in ``libjoshua_hip.so`` (hand-written
HIP for gfx950, C ABI declared in ``include/joshua_hip.h``); ``joshua_amd.capi``
binds it with ctypes and raises if the library is missing."""

__all__ = ["capi", "synth"]
