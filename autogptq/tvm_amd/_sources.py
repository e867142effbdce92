"""The sources the two in-tree libraries are built from, and their digest."""
from __future__ import annotations

import hashlib
import os

CSRC = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc")
SOURCES = ["gptq_stream.hip", "gptq_grouped.hip", "gptq_dequant.hip", "gptq_static.hip", "gptq_probe.hip", "gptq_tiled.hip", "gptq_tiled_decode.hip", "gptq_tiled_decode16.hip", "gptq_dispatch.cpp", "gptq_capi.cpp"]
HEADERS = ["gptq_unpack.h", "gptq_internal.h", "gptq_device.h", "gptq_tiled_common.h", os.path.join("..", "..", "..", "include", "gptq_hip.h"),
           "binding.cpp"]   # (hashed with the rest: both libraries carry one build id)
# Compiler options of single sources.  The decode kernels keep the four result registers of their small matrix
# instructions in ordinary vector registers: left to itself the compiler puts them into accumulation registers
# for the workgroups of four waves and copies them back for every epilogue.  The same kernels take their first sixteen
# dwords of arguments preloaded into scalar registers.
EXTRA_FLAGS = {
    "gptq_tiled_decode.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form", "-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gptq_tiled_decode16.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gptq_tiled.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
    "gptq_dequant.hip": ["-mllvm", "-amdgpu-kernarg-preload-count=16"],
}


def source_hash() -> str:
    """Digest of every source and header the library is built from; the library reports the digest it
    was built with (gptq_hip_build_id), so a library older than its sources is noticed when it is loaded."""
    h = hashlib.sha256()
    for name in sorted(SOURCES + HEADERS):
        with open(os.path.join(CSRC, name), "rb") as f:
            h.update(name.encode() + b"\0" + f.read() + b"\0")
    h.update(repr(sorted(EXTRA_FLAGS.items())).encode())
    return h.hexdigest()[:16]


