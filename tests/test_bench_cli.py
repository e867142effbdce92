"""bench.py's command-line contract, as far as it can be checked without a GPU."""
import json
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def run(*args, env=None):
    e = dict(os.environ)
    e.update(env or {})
    return subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), *args], capture_output=True, text=True,
                          cwd=ROOT, env=e, timeout=300)


def test_more_than_one_gpu_is_refused_with_a_message():
    r = run("--gpus", "2")
    assert r.returncode == 2 and "ONE GPU" in r.stderr and r.stdout.strip() == ""
    r = run(env={"WORLD_SIZE": "4"})
    assert r.returncode == 2 and "ONE GPU" in r.stderr


def test_workload_table_covers_the_baseline_configurations():
    sys.path.insert(0, ROOT)
    import bench

    names = set(bench.WORKLOADS)
    assert bench.DEFAULT_WORKLOAD in names
    bits, K, N, gs, act, M = bench.WORKLOADS[bench.DEFAULT_WORKLOAD]
    assert (bits, K, N, gs, act, M) == (3, 4096, 11008, 128, True, 1)      # the headline configuration
    assert bench.WORKLOADS["c1-int4-4096x4096-m1"] == (4, 4096, 4096, 128, False, 1)  # configs[0]
    assert any(v[5] == 128 and v[4] for v in bench.WORKLOADS.values())     # act-order GEMM at M = 128
    assert any(v[3] == -1 and v[1] == 36864 for v in bench.WORKLOADS.values())  # OPT-66B long K
    for name in bench.SECONDARY_WORKLOADS:
        assert name in names
    # the measured-traffic table names workloads that exist and the profile summaries its figures come from
    import json
    with open(bench.TRAFFIC_FILE) as f:
        table = json.load(f)
    for name, e in table.items():
        assert name in names
        assert os.path.exists(os.path.join(ROOT, e["source"])), e["source"]
        assert e["fetch_bytes"] > 0 and e["write_bytes"] >= 0
    total, source = bench.measured_traffic("c2-int3-4096x11008-act-m1", table["c2-int3-4096x11008-act-m1"]["plan_kernel"])
    assert total == table["c2-int3-4096x11008-act-m1"]["fetch_bytes"] + table["c2-int3-4096x11008-act-m1"]["write_bytes"]
    assert source.startswith("profiles/")
    assert bench.measured_traffic("c2-int3-4096x11008-act-m1", 99) == (None, None)   # another kernel than the one measured
