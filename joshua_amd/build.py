"""Builds the native libraries in-tree: libjoshua_hip.so (HIP, gfx950) and the
host-only synthetic-input library."""
from __future__ import annotations

import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
HIP_LIB = os.path.join(HERE, "libjoshua_hip.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
    # keep the compiler from forming packed-f32 instructions out of scalar float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the leading kernel arguments arrive in scalar registers with the wave instead of by a scalar load
    # from memory at its entry (0.4 us sooner to the first global load of a kernel that starts cold)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
]


def hip_sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def build_hip(verbose: bool = False) -> str:
    cmd = ["hipcc", *HIPCC_FLAGS, "-o", HIP_LIB, *hip_sources()]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed:\n{err}")
    if verbose and err.strip():
        print(err)
    return HIP_LIB


CALIB_SRC = os.path.join(HERE, "calib", "copy_kernel.hip")
CALIB_BIN = os.path.join(HERE, "calib", "copy_kernel")


PROBE_SRC = os.path.join(HERE, "calib", "read_probe.hip")
PROBE_BIN = os.path.join(HERE, "calib", "read_probe")
MIX_SRC = os.path.join(HERE, "calib", "gemm_mix_probe.hip")
MIX_BIN = os.path.join(HERE, "calib", "gemm_mix_probe")


def build_calibration() -> str:
    """The copy kernel that calibrates the FETCH_SIZE / WRITE_SIZE counters, the plain-read probe that gives
    the floor of one launch over a matrix of the benchmark's size, and the probe that runs the int8 GEMM's
    instruction mix of a super-block iteration with nothing else around it."""
    for src, out in ((CALIB_SRC, CALIB_BIN), (PROBE_SRC, PROBE_BIN), (MIX_SRC, MIX_BIN)):
        res = subprocess.run(["hipcc", "--offload-arch=gfx950", "-O3", "-o", out, src], capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f"hipcc failed:\n{res.stderr}")
    return CALIB_BIN


def build_all(verbose: bool = False) -> None:
    """The library and the synthetic-data helper: what tests, smoke and the benchmark load.  The counter
    calibration program is a profiling aid, built on request (`python -m joshua_amd.build --calibration`)."""
    from . import synth
    build_hip(verbose)
    synth.build()


if __name__ == "__main__":
    import sys
    if "--calibration" in sys.argv[1:]:
        print("built", build_calibration())
    else:
        build_all(verbose=True)
        print("built", HIP_LIB)
