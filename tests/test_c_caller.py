"""The C ABI from plain C: tests/host/c_caller.c is compiled with gcc against include/gptq_hip.h and the built
library (no torch, no C++), run on the GPU, and its three results (checkpoint tensors, channel-sorted copy,
tiled copy) are compared with the CPU oracle."""
import os
import shutil
import subprocess

import numpy as np
import pytest
import torch

from autogptq.tvm_amd import _lib
from tests.parity_util import assert_close, assert_tight, expected_output, layer

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "autogptq", "tvm_amd", "csrc")


def build_caller(tmp_path):
    gcc = shutil.which("gcc")
    if gcc is None or not os.path.exists("/opt/rocm/include/hip/hip_runtime_api.h"):
        pytest.skip("gcc or the HIP runtime headers are missing")
    exe = tmp_path / "c_caller"
    subprocess.check_call([gcc, "-std=c99", "-O1", "-Wall", "-Werror", "-D__HIP_PLATFORM_AMD__=1", "-I", os.path.join(ROOT, "include"),
                           "-I", "/opt/rocm/include", os.path.join(ROOT, "tests", "host", "c_caller.c"), "-o", str(exe),
                           "-L", CSRC, "-lgptq_hip", "-L", "/opt/rocm/lib", "-lamdhip64",
                           f"-Wl,-rpath,{CSRC}", "-Wl,-rpath,/opt/rocm/lib"])
    return exe


def test_c_caller_compiles_against_the_header(tmp_path):
    """gcc -std=c99 -Wall -Werror: the header is C, and every entry point the caller uses links."""
    _lib.lib()
    build_caller(tmp_path)


@pytest.mark.gpu
@pytest.mark.parametrize("bits,K,N,gs,act,M", [(4, 1024, 416, 128, True, 1), (3, 1024, 416, 128, True, 8),
                                                (3, 2048, 1056, 256, True, 40), (4, 384, 64, 64, False, 3),
                                                (4, 4096, 352, 128, True, 130)])
def test_c_caller_matches_the_oracle(tmp_path, bits, K, N, gs, act, M):
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    exe = build_caller(tmp_path)
    L = layer(3000 + K + M, K, N, bits, gs, act, M=M, bias=True)
    inp, out = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(inp, "wb") as f:
        f.write(np.array([M, K, N, bits, gs, int(act)], dtype=np.int32).tobytes())
        for name in ("qweight", "qzeros", "scales", "g_idx", "x", "bias"):
            f.write(L[name].contiguous().numpy().tobytes())
    r = subprocess.run([str(exe), str(inp), str(out)], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert r.returncode == 0 and r.stdout.startswith("ok "), r.stdout
    y = torch.from_numpy(np.fromfile(out, dtype=np.float16).reshape(3, M, N).copy())
    want = expected_output(L)
    for i, what in enumerate(("gptq_hip_gemm", "gptq_hip_gemm_sorted", "gptq_hip_gemm_tiled")):
        assert_close(y[i], want, f"C caller, {what}")
        assert_tight(y[i], want, f"C caller, {what}")
