"""The build writes registers, scratch and spills per kernel; no shipped kernel may
spill (a few registers over the 256 of two-waves-per-SIMD occupancy cost the int3 GEMM 50 % once)."""
import json
import os

import pytest

from autogptq.tvm_amd import build

SAMPLE = """
a.hip:47:1: remark: Function Name: _ZN4gptq1kEv [-Rpass-analysis=kernel-resource-usage]
   47 | {
      | ^
a.hip:47:1: remark:     TotalSGPRs: 14 [-Rpass-analysis=kernel-resource-usage]
a.hip:47:1: remark:     VGPRs: 250 [-Rpass-analysis=kernel-resource-usage]
a.hip:47:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:47:1: remark:     ScratchSize [bytes/lane]: 28 [-Rpass-analysis=kernel-resource-usage]
a.hip:47:1: remark:     Occupancy [waves/SIMD]: 2 [-Rpass-analysis=kernel-resource-usage]
a.hip:47:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:47:1: remark:     VGPRs Spill: 6 [-Rpass-analysis=kernel-resource-usage]
"""


def test_parse_resource_remarks():
    r = build.parse_resource_remarks(SAMPLE)
    assert r == {"_ZN4gptq1kEv": {"vgprs": 250, "agprs": 0, "scratch": 28, "occupancy": 2, "sgpr_spill": 0,
                                  "vgpr_spill": 6}}


def test_hot_path_kernels_do_not_spill():
    if not os.path.exists(build.REPORT):
        pytest.skip("library was built without the resource report")
    with open(build.REPORT) as f:
        report = json.load(f)
    names = list(report)
    assert any("stream_kernel" in n for n in names) and any("grouped_kernel" in n for n in names)
    for name, r in report.items():
        assert r.get("vgpr_spill", 0) == 0 and r.get("scratch", 0) == 0, (name, r)   # every shipped kernel
        if "stream_kernel" in name or "stream_direct" in name or "grouped_kernel" in name:
            assert r.get("occupancy", 0) >= 2, (name, r)   # two waves per SIMD is what these designs assume
