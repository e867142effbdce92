"""Builds csrc/gptq_unpack.h for the host with ROCm's clang and checks the register-level
unpack (the fp16 magic-number trick the kernels use) against plain bit extraction."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _clang():
    for c in ("/opt/rocm/llvm/bin/clang++", "/opt/rocm/lib/llvm/bin/clang++", shutil.which("amdclang++"),
              shutil.which("clang++")):
        if c and os.path.exists(c):
            return c
    return None


def test_magic_unpack_matches_bit_extraction(tmp_path):
    cxx = _clang()
    if cxx is None:
        pytest.skip("no clang++ with _Float16 vector support found")
    exe = tmp_path / "unpack_check"
    subprocess.check_call([cxx, "-std=c++17", "-O1", "-I", os.path.join(ROOT, "autogptq", "tvm_amd", "csrc"),
                           os.path.join(ROOT, "tests", "host", "unpack_check.cpp"), "-o", str(exe)])
    out = subprocess.run([str(exe)], stdout=subprocess.PIPE, text=True)
    assert out.returncode == 0, out.stdout
    assert out.stdout.startswith("ok ")
    # the Python mirror of the slot tables (used by the load-time channel sort) matches the header
    from autogptq.tvm_amd import _slots

    lines = {l.split()[0]: [int(v) for v in l.split()[1:]] for l in out.stdout.splitlines()[1:]}
    assert lines["slot4"] == _slots.CODE_OF_SLOT4
    assert lines["slot3"] == _slots.CODE_OF_SLOT3
    assert lines["slot8"] == _slots.CODE_OF_SLOT8
    assert lines["slot2"] == _slots.CODE_OF_SLOT2
    # the tiled format's permutation per width, as the kernels' codec states it
    for bits in (2, 3, 4, 8):
        assert lines[f"field{bits}"] == _slots.lane_field_of_position(bits)
        assert lines[f"base{bits}"] == _slots.BASE_OF_POSITION[bits]
