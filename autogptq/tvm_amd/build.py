"""Builds the C-ABI shared library of HIP kernels for gfx950, in-tree, with hipcc.

``python -m autogptq.tvm_amd.build`` compiles ``csrc/*.hip`` and ``csrc/*.cpp`` into
``csrc/libgptq_hip.so``.  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(CSRC, "libgptq_hip.so")
SOURCES = ["gptq_gather.hip", "gptq_stream.hip", "gptq_grouped.hip", "gptq_dequant.hip", "gptq_dispatch.cpp", "gptq_capi.cpp"]
HEADERS = ["gptq_unpack.h", "gptq_internal.h", "gptq_device.h", os.path.join("..", "..", "..", "include", "gptq_hip.h")]


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH)")


def flags() -> list:
    return [
        "--offload-arch=gfx950",
        "-O3",
        "-std=c++17",
        "-fPIC",
        "-shared",
        # keep the compiler from forming packed-fp32 instructions
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    ]


def is_stale() -> bool:
    if not os.path.exists(LIB):
        return True
    t = os.path.getmtime(LIB)
    deps = [os.path.join(CSRC, s) for s in SOURCES + HEADERS]
    return any(os.path.getmtime(d) > t for d in deps)


def build(verbose: bool = False) -> str:
    cmd = [hipcc()] + flags() + ["-o", LIB] + [os.path.join(CSRC, s) for s in SOURCES]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "is not a recognized feature" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
