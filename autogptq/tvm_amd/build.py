"""Builds the C-ABI shared library of HIP kernels for gfx950, in-tree, with hipcc, and the torch operator
library on top of it.

``python -m autogptq.tvm_amd.build`` compiles ``csrc/*.hip`` and ``csrc/*.cpp`` into
``csrc/libgptq_hip.so`` (no torch in it), then ``csrc/binding.cpp`` against the installed torch headers into
``csrc/libgptq_hip_torch.so`` (``torch.ops.gptq_hip.*``).  hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import json
import os
import shutil
import subprocess
import sys

from ._sources import CSRC, EXTRA_FLAGS, HEADERS, SOURCES, source_hash  # noqa: F401

LIB = os.path.join(CSRC, "libgptq_hip.so")
BINDING_LIB = os.path.join(CSRC, "libgptq_hip_torch.so")


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", shutil.which("hipcc")):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked at $HIPCC, /opt/rocm/bin/hipcc and PATH)")


def flags() -> list:
    return [
        "--offload-arch=gfx950",
        "-O3",
        "-std=c++20",
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


REPORT = os.path.join(CSRC, "kernel_resources.json")


def parse_resource_remarks(text: str) -> dict:
    """{kernel symbol: {"vgprs", "agprs", "scratch", "vgpr_spill", "sgpr_spill", "occupancy"}} from the
    compiler's -Rpass-analysis=kernel-resource-usage remarks."""
    keys = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch", "VGPRs Spill": "vgpr_spill",
            "SGPRs Spill": "sgpr_spill", "Occupancy [waves/SIMD]": "occupancy"}
    res, cur = {}, None
    for line in text.splitlines():
        if "remark:" not in line:
            continue
        body = line.split("remark:", 1)[1].split("[-Rpass", 1)[0].strip()
        if body.startswith("Function Name:"):
            cur = res.setdefault(body.split(":", 1)[1].strip(), {})
        elif cur is not None and ":" in body:
            k, v = body.rsplit(":", 1)
            if k.strip() in keys:
                cur[keys[k.strip()]] = int(v)
    return res


def _compile_one(src: str, obj: str, build_id: str):
    cmd = [hipcc()] + [f for f in flags() if f != "-shared"] + EXTRA_FLAGS.get(os.path.basename(src), []) + [
        f'-DGPTQ_HIP_BUILD_ID="{build_id}"', "-Rpass-analysis=kernel-resource-usage", "-c", "-o", obj, src]
    return subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)


def build_binding(build_id: str) -> str:
    """binding.cpp -> libgptq_hip_torch.so: host C++ only (no device code), against torch's headers and
    libraries, linked to libgptq_hip.so beside it."""
    import torch
    from torch.utils import cpp_extension as ce

    inc = [f"-I{d}" for d in ce.include_paths()] + ["-I/opt/rocm/include", f"-I{os.path.join(CSRC, '..', '..', '..', 'include')}"]
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [hipcc(), "-x", "c++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", f'-DGPTQ_HIP_BUILD_ID="{build_id}"',
           "-Wno-deprecated-declarations"] + inc + [
        os.path.join(CSRC, "binding.cpp"), "-o", BINDING_LIB, f"-L{CSRC}", "-lgptq_hip", f"-L{tlib}", "-lc10", "-lc10_hip",
        "-ltorch_cpu", "-ltorch_hip", "-ltorch", "-Wl,-rpath,$ORIGIN"]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if r.returncode != 0:
        raise RuntimeError("building the torch operator library failed:\n" + r.stdout)
    return BINDING_LIB


def build(verbose: bool = False, jobs: int = 0) -> str:
    """Compiles every source to an object file (in parallel, at most 8 at a time) and links the library."""
    from concurrent.futures import ThreadPoolExecutor

    build_id = source_hash()
    objdir = os.path.join(CSRC, "build")
    os.makedirs(objdir, exist_ok=True)
    pairs = [(os.path.join(CSRC, s), os.path.join(objdir, os.path.splitext(s)[0] + ".o")) for s in SOURCES]
    jobs = jobs or min(8, len(pairs), os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        procs = list(pool.map(lambda so: _compile_one(so[0], so[1], build_id), pairs))
    text = "\n".join(p.stdout for p in procs)
    report = parse_resource_remarks(text)
    noise = ("is not a recognized feature", "remark:", "-Rpass-analysis")
    lines, skip = [], 0
    for l in text.splitlines():
        if skip:          # the two source-echo lines that follow every remark
            skip -= 1
            continue
        if "remark: Function Name" in l:
            skip = 2
        if not any(n in l for n in noise):
            lines.append(l)
    out = "\n".join(lines)
    if any(p.returncode != 0 for p in procs):
        raise RuntimeError("hipcc failed:\n" + out)
    link = subprocess.run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + [o for _, o in pairs],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if link.returncode != 0:
        raise RuntimeError("link failed:\n" + link.stdout)
    build_binding(build_id)
    with open(REPORT, "w", encoding="utf-8") as f:   # registers, scratch and spills per kernel
        json.dump(report, f, indent=1, sort_keys=True)
    spilled = sorted(k for k, v in report.items() if v.get("vgpr_spill", 0) or v.get("scratch", 0))
    if verbose:
        if out.strip():
            print(out)
        for k in spilled:
            print(f"note: {k} spills {report[k].get('vgpr_spill', 0)} VGPRs ({report[k].get('scratch', 0)} B scratch/lane)")
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
    sys.exit(0)
