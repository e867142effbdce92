#!/usr/bin/env python3
"""Benchmark of the GPTQ QuantLinear hot path on one MI355X.

Default workload: the headline configuration of the reference's benchmarks -- 3-bit GEMV, M=1, K=4096, N=11008, group_size=128,
desc_act=True (g_idx from a random permutation), synthetic seeded tensors.  One "step" is one
call of the C-ABI entry point that ``QuantLinear.forward`` makes for that shape, on tensors already
resident in HBM: ``gptq_hip_gemm_sorted`` for decode sizes on activation-order layers (the layer
as the module holds it after its one-time load preparation, the channel sort),
``gptq_hip_gemm_tiled`` where the module routes to its copy in the tiled format (prompt sizes; decode
sizes of layers up to 8192 columns wide), ``gptq_hip_gemm`` otherwise; ``--unprepared`` times
``gptq_hip_gemm`` on the checkpoint's own tensors instead, and the default run reports that figure
too under ``timing.unprepared_us``.  Steps rotate
over enough distinct weight copies to exceed twice the 256 MB Infinity Cache, so every step
streams its packed weights from HBM (cache-cold).

Prints ONE JSON line (see the keys below).  ``roofline.achieved`` is algorithmic bytes (packed
qweight only, K*N*bits/8) or flops (2*M*K*N) per launch divided by the average launch duration
measured here with HIP events on the launch stream.  ``cpu_baseline`` times the CPU oracle (the
restatement of the reference's torch path) on this box's host cores.

Other workloads: ``--workload NAME`` (see WORKLOADS), ``--sweep`` adds a table of all of them
under "sweep" in the same JSON line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import statistics
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16
INFINITY_CACHE_BYTES = 256 << 20

# name -> (bits, K, N, group_size, desc_act, M)
WORKLOADS = {
    "c1-int4-4096x4096-m1": (4, 4096, 4096, 128, False, 1),
    "c2-int3-4096x11008-act-m1": (3, 4096, 11008, 128, True, 1),
    "int4-4096x11008-act-m1": (4, 4096, 11008, 128, True, 1),
    "c3-int4-4096x4096-m1": (4, 4096, 4096, 128, False, 1),
    "c3-int4-4096x11008-m1": (4, 4096, 11008, 128, False, 1),
    "c3-int4-4096x11008-m2": (4, 4096, 11008, 128, False, 2),
    "c3-int4-4096x11008-m4": (4, 4096, 11008, 128, False, 4),
    "c3-int4-4096x11008-m8": (4, 4096, 11008, 128, False, 8),
    "c3-int4-11008x4096-m1": (4, 11008, 4096, 128, False, 1),
    "c3-int4-11008x4096-m8": (4, 11008, 4096, 128, False, 8),
    "int3-11008x4096-act-m1": (3, 11008, 4096, 128, True, 1),
    "int4-11008x4096-act-m1": (4, 11008, 4096, 128, True, 1),
    "int3-4096x4096-act-m1": (3, 4096, 4096, 128, True, 1),
    "int3-4096x11008-m1": (3, 4096, 11008, 128, False, 1),
    # q/k/v and gate/up of a 4096-wide block as one product each (fused.fuse_shared_input_layers)
    "qkv-int4-4096x12288-act-m1": (4, 4096, 12288, 128, True, 1),
    "qkv-int3-4096x12288-act-m1": (3, 4096, 12288, 128, True, 1),
    "gateup-int4-4096x22016-act-m1": (4, 4096, 22016, 128, True, 1),
    "gateup-int3-4096x22016-act-m1": (3, 4096, 22016, 128, True, 1),
    "c4-int4-4096x11008-act-m16": (4, 4096, 11008, 128, True, 16),
    "c4-int4-4096x11008-act-m64": (4, 4096, 11008, 128, True, 64),
    "c4-int4-4096x11008-act-m128": (4, 4096, 11008, 128, True, 128),
    "c4-int4-4096x11008-act-m256": (4, 4096, 11008, 128, True, 256),
    "c4-int4-4096x11008-act-m1024": (4, 4096, 11008, 128, True, 1024),
    "c4-int3-4096x11008-act-m1024": (3, 4096, 11008, 128, True, 1024),
    "c4-int3-4096x11008-act-m128": (3, 4096, 11008, 128, True, 128),
    "int4-4096x11008-m128": (4, 4096, 11008, 128, False, 128),
    "int4-4096x11008-m256": (4, 4096, 11008, 128, False, 256),
    "c4-int4-11008x4096-act-m128": (4, 11008, 4096, 128, True, 128),
    "c4-int3-11008x4096-act-m128": (3, 11008, 4096, 128, True, 128),
    "c5-int3-9216x9216-g1-m1": (3, 9216, 9216, -1, True, 1),
    "c5-int3-9216x36864-g1-m1": (3, 9216, 36864, -1, True, 1),
    "c5-int3-36864x9216-g1-m1": (3, 36864, 9216, -1, True, 1),
    "c5-int3-9216x36864-g1-m32": (3, 9216, 36864, -1, True, 32),
    # larger layers, where the fixed cost of a launch weighs less
    "int4-9216x36864-g1-m1": (4, 9216, 36864, -1, True, 1),
    "int4-8192x28672-m1": (4, 8192, 28672, 128, False, 1),
    "int3-8192x28672-act-m1": (3, 8192, 28672, 128, True, 1),
    # the other widths of the format: fused on the tiled format only
    "int8-4096x11008-act-m1": (8, 4096, 11008, 128, True, 1),
    "int2-4096x11008-act-m1": (2, 4096, 11008, 128, True, 1),
    "int8-4096x11008-act-m128": (8, 4096, 11008, 128, True, 128),
    "int2-4096x11008-act-m128": (2, 4096, 11008, 128, True, 128),
}
DEFAULT_WORKLOAD = "c2-int3-4096x11008-act-m1"
# timed in the default run next to the headline: the int4 decode product and the M = 128 products of the
# same 4096 x 11008 activation-order layer (the metric is quoted on all of them)
SECONDARY_WORKLOADS = ("int4-4096x11008-act-m1", "c4-int4-4096x11008-act-m128", "c4-int3-4096x11008-act-m128")

# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (each scaled by what the same
# counter reads for a plain 256 MiB device copy): profiles/traffic.json holds, per workload, the bytes, the
# kernel they were measured on and the summary under profiles/ they come from.  A workload without an entry,
# or whose entry names another kernel plan than the one timed here, reports null.
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "traffic.json")


def measured_traffic(workload: str, plan_kernel: int):
    try:
        with open(TRAFFIC_FILE, encoding="utf-8") as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None, None
    e = table.get(workload)
    if not e or e.get("plan_kernel") != plan_kernel:
        return None, None
    return int(e["fetch_bytes"]) + int(e["write_bytes"]), e.get("source")


def build_case(name: str, dev, kernel: int = 0, split_k: int = 0, waves_n: int = 0, prepared=None):
    """prepared: the layer as QuantLinear holds it after its one-time preparation: "sorted" (channels of
    an activation-order layer sorted by group, run through gptq_hip_gemm_sorted), "tiled" (the tiled
    format, run through gptq_hip_gemm_tiled), or None (the checkpoint's tensors, gptq_hip_gemm);
    prepared_mode(name) is the module's own choice."""
    from autogptq.tvm_amd import _lib, ops
    from autogptq.tvm_amd.pack import sort_channels_by_group, synth_layer

    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    L = synth_layer(2000 + sorted(WORKLOADS).index(name), K, N, bits, gs, desc_act, M=M)
    wbytes = K * N * bits // 8
    copies = max(2, -(-2 * INFINITY_CACHE_BYTES // wbytes))
    gen = torch.Generator().manual_seed(99)
    case = {
        "name": name, "bits": bits, "K": K, "N": N, "gs": gs, "desc_act": desc_act, "M": M, "L": L,
        "qzeros": L["qzeros"].to(dev), "scales": L["scales"].to(dev),
        "g_idx": L["g_idx"].to(dev) if desc_act else None,
        "x": L["x"].to(dev), "y": torch.empty((M, N), dtype=torch.float16, device=dev),
        "wbytes": wbytes, "flops": 2 * M * K * N, "kmap": None, "tiled": None, "prepared": prepared,
    }
    qweights = []
    for c in range(copies):
        # copy 0 is the seeded layer; the others are distinct random packed words (every int32 pattern is a
        # valid block of codes)
        q = L["qweight"].to(dev) if c == 0 else torch.randint(
            -(1 << 31), (1 << 31) - 1, L["qweight"].shape, generator=gen, dtype=torch.int64).to(torch.int32).to(dev)
        if prepared == "tiled":
            # (every copy brings its own scale / zero words and channel maps, as every layer of a model does)
            qtile, sz, xsrc, kinv = ops.tile_prepare(q, case["qzeros"], case["scales"], case["g_idx"], bits, gs)
            case.setdefault("tiled_copies", []).append((sz, xsrc if desc_act else None, kinv if desc_act else None))
            if c == 0:
                case["tiled"] = case["tiled_copies"][0]
            q = qtile
        qweights.append(q)
    case["qweights"] = qweights
    if prepared == "sorted":
        qweights[0], case["kmap"] = sort_channels_by_group(qweights[0], case["g_idx"], bits, gs)
        case["g_idx"] = None
        desc_act = False  # the plan is that of contiguous groups
    # the layer's other tensors, one set per copy as well (qzeros, scales, and g_idx or the sorted copy's map)
    g_or_map = case["kmap"] if case["kmap"] is not None else case["g_idx"]
    case["aux_copies"] = [(case["qzeros"], case["scales"], g_or_map)] + [
        (case["qzeros"].clone(), case["scales"].clone(), g_or_map.clone() if g_or_map is not None else None)
        for _ in range(copies - 1)]
    if prepared == "tiled":
        plan = _lib.select_tiled(M, K, N, bits, gs)
    elif prepared == "sorted" and not (kernel or split_k or waves_n):
        plan = ops.sorted_plan(M, K, N, bits, gs)
    elif kernel or split_k or waves_n:
        if not kernel:
            kernel = _lib.select(M, K, N, bits, gs, desc_act).kernel
        plan = _lib.plan_for(kernel, M, K, N, bits, gs, desc_act, split_k, waves_n)
    else:
        plan = _lib.select(M, K, N, bits, gs, desc_act)
    case["plan"] = plan
    ws_bytes = plan.workspace_bytes
    if prepared == "sorted":   # kernels that want x in the sorted order find it behind the plan's own bytes
        ws_bytes = max(ws_bytes, _lib.lib().gptq_hip_sorted_workspace_bytes(M, K, N, bits, gs))
    case["ws_bytes"] = ws_bytes
    case["ws"] = torch.zeros(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
    return case


ENTRY = {None: "gptq_hip_gemm_plan", "sorted": "gptq_hip_gemm_sorted", "tiled": "gptq_hip_gemm_tiled"}
PREPARED_NOTE = {None: None, "sorted": "input channels sorted by group once at load",
                 "tiled": "layer re-laid once at load into the tiled format (gptq_hip_tile_prepare)"}


def plain_applies(name: str) -> bool:
    """The kernels on the checkpoint layout (and its sorted copy) cover 3 and 4 bits."""
    from autogptq.tvm_amd import ops

    return WORKLOADS[name][0] in ops.FUSED_BITS


def sorted_applies(name: str) -> bool:
    from autogptq.tvm_amd import ops

    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    G = 1 if gs == -1 else -(-K // gs)
    if not plain_applies(name):
        return False
    return bool(desc_act and G > 1 and M <= ops.SORTED_MAX_ROWS and ops.sorted_plan(M, K, N, bits, gs) is not None)


def tiled_applies(name: str) -> bool:
    from autogptq.tvm_amd.pack import tiled_qualifies

    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    return tiled_qualifies(K, N, bits, gs)


def prepared_mode(name: str):
    """The prepared copy QuantLinear.forward uses for this workload (qlinear.py: _product), or None."""
    from autogptq.tvm_amd import ops

    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    one_group = gs == -1 or gs >= K
    if tiled_applies(name) and (not plain_applies(name) or ops.tiled_wins(M, K, N, desc_act and not one_group, bits,
                                                                           one_group=one_group)):
        return "tiled"
    return "sorted" if sorted_applies(name) else None


def make_step(case, dev):
    """Returns step(i): one call of the case's entry point on weight copy i (pre-marshalled arguments)."""
    from autogptq.tvm_amd import _lib

    lib = _lib.lib()
    vp = ctypes.c_void_p
    ptr = lambda t: vp(t.data_ptr()) if t is not None else None
    qws = [vp(q.data_ptr()) for q in case["qweights"]]
    x, y = ptr(case["x"]), ptr(case["y"])
    ws, wsb = (ptr(case["ws"]) if case["ws_bytes"] else None), case["ws_bytes"]
    M, K, N, bits, gs = case["M"], case["K"], case["N"], case["bits"], case["gs"]
    planp = ctypes.byref(case["plan"])
    n = len(qws)
    if case["prepared"] == "tiled":
        aux = [tuple(ptr(t) for t in c) for c in case["tiled_copies"]]

        def step(i, stream):
            sz, xsrc, kinv = aux[i % n]
            rc = lib.gptq_hip_gemm_tiled(x, qws[i % n], sz, xsrc, kinv, None, y, ws, wsb, M, K, N, bits, gs, planp, stream)
            if rc != 0:
                raise RuntimeError(f"gptq_hip_gemm_tiled failed: {_lib.strerror(rc)}")

        return step
    fn = lib.gptq_hip_gemm_sorted if case["kmap"] is not None else lib.gptq_hip_gemm_plan
    aux = [tuple(ptr(t) for t in c) for c in case["aux_copies"]]

    def step(i, stream):
        qz, sc, g = aux[i % n]
        rc = fn(x, qws[i % n], qz, sc, g, None, y, ws, wsb, M, K, N, bits, gs, planp, stream)
        if rc != 0:
            raise RuntimeError(f"gptq_hip_gemm failed: {_lib.strerror(rc)}")

    return step


_scrub = {}


def scrub_cache(dev):
    """Reads a buffer of twice the Infinity Cache, so that nothing a later step reads is still cached.  (Reads,
    not writes: a cache left full of dirty lines drains into HBM under the first ~250 MB that the timed steps
    read, and they pay for that traffic: 20 steps of the headline measured 8.9 us each behind a zero fill, 7.3
    behind this read, 6.9 for 200 steps either way.)"""
    if dev not in _scrub:
        _scrub[dev] = torch.zeros(2 * INFINITY_CACHE_BYTES // 8, dtype=torch.int64, device=dev)
        torch.cuda.synchronize(dev)
    _scrub[dev].sum()


def time_case(case, dev, steps: int, warmup: int):
    """Average duration of one step in microseconds: K steps captured once in a HIP graph and
    replayed inside one event-bracketed region (no host launch cost between the kernels; reported as
    ``graph_us`` and as ``us``), plus the same K steps launched eagerly (``eager_us``).  The W warm-up steps
    run right in front of the timed ones, on the same stream with nothing in between, so that the K steps
    start on a busy GPU (the first steps behind an idle or scrubbed GPU take ~2 us longer each: 5 steps
    measure 8.8 us, steps 6 to 20 of 20 measure 7.0).  The weight copy of step i is (warmup + i) mod copies,
    continuing the warm-up's rotation, and the cache is scrubbed before the warm-up of every timed region, so
    no timed step finds its weights cached."""
    step = make_step(case, dev)
    stream = torch.cuda.Stream(device=dev)
    res = {}
    with torch.cuda.stream(stream):
        sp = ctypes.c_void_p(stream.cuda_stream)
        for i in range(warmup):       # (first calls: lazy initialisation of the runtime for these kernels)
            step(i, sp)
        stream.synchronize()
        # eager
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize(dev)
        scrub_cache(dev)
        for i in range(warmup):
            step(i, sp)
        e0.record(stream)
        for i in range(steps):
            step(warmup + i, sp)
        e1.record(stream)
        torch.cuda.synchronize(dev)
        res["eager_us"] = e0.elapsed_time(e1) * 1e3 / steps
    # graph replay
    try:
        g, g_warm = torch.cuda.CUDAGraph(), torch.cuda.CUDAGraph()
        if warmup > 0:
            with torch.cuda.graph(g_warm, stream=stream):
                spg = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
                for i in range(warmup):
                    step(i, spg)
        with torch.cuda.graph(g, stream=stream):
            spg = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
            for i in range(steps):
                step(warmup + i, spg)
        g.replay()
        torch.cuda.synchronize(dev)
        times = []
        for _ in range(3):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize(dev)
            # scrub, W warm-up steps, then the K timed steps, queued back to back
            scrub_cache(dev)
            if warmup > 0:
                g_warm.replay()
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize(dev)
            times.append(e0.elapsed_time(e1) * 1e3 / steps)
        res["graph_us"] = min(times)
    except Exception as exc:  # graph capture unavailable: report the eager figure only
        res["graph_error"] = repr(exc)[:200]
    res["us"] = res.get("graph_us", res["eager_us"])
    return res


def check_case(case, dev):
    """The timed path's output against the oracle, for the first weight copy."""
    from oracle import c_oracle

    step = make_step(case, dev)
    step(0, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    torch.cuda.synchronize(dev)
    L = case["L"]
    w16 = torch.from_numpy(c_oracle.dequant(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(),
                                            L["g_idx"].numpy(), case["bits"]).copy())
    want = L["x"].float() @ w16.float()
    got = case["y"].float().cpu()
    err = (got - want).abs()
    ok = bool((err <= 1e-2 + 1e-2 * want.abs()).all())
    return ok, float(err.max())


def summarize(case, t):
    us = t["us"]
    out = {"workload": case["name"], "us": round(us, 3)}
    out.update({k: (round(v, 3) if isinstance(v, float) else v) for k, v in t.items() if k != "us"})
    out["weight_GBps"] = round(case["wbytes"] / us * 1e-3, 1)
    out["hbm_frac"] = round(case["wbytes"] / us * 1e-3 / HBM_PEAK_GBS, 4)
    out["TFLOPs"] = round(case["flops"] / us * 1e-6, 2)
    out["mfma_frac"] = round(case["flops"] / us * 1e-6 / MFMA_FP16_PEAK_TFLOPS, 4)
    out["plan"] = {k: v for k, v in case["plan"].as_dict().items()
                   if k in ("kernel", "row_tiles", "waves_n", "waves_k", "split_k", "grid_x", "grid_y", "grid_z")}
    return out


def roofline_of(name: str, s: dict) -> dict:
    """The roofline object of one timed workload: HBM-bound for decode sizes (M <= 8), MFMA-bound above."""
    M = WORKLOADS[name][5]
    traffic, source = measured_traffic(name, s["plan"]["kernel"])
    if M <= 8:
        r = {"bound": "hbm", "achieved": s["weight_GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": s["hbm_frac"]}
    else:
        r = {"bound": "mfma", "achieved": s["TFLOPs"], "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
             "frac": s["mfma_frac"], "hbm_frac": s["hbm_frac"]}
    r["traffic"] = traffic
    r["traffic_source"] = source
    return r


def cpu_baseline(case, budget_s: float = 20.0):
    """The reference's CPU path (oracle restatement of qlinear.py:198-245: unpack + gather + dequant
    + fp16 matmul on every call) on this box's host cores."""
    from oracle import gptq_oracle as orc

    L = case["L"]
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1))
    torch.set_num_threads(threads)
    args = (L["x"], L["qweight"], L["qzeros"], L["scales"], L["g_idx"], None, case["bits"])
    t0 = time.perf_counter()
    orc.forward_ref(*args)
    first = time.perf_counter() - t0
    n = max(3, min(10, int(budget_s / max(first, 1e-3)) - 1))
    ts = []
    for _ in range(n):
        t0 = time.perf_counter()
        orc.forward_ref(*args)
        ts.append(time.perf_counter() - t0)
    med = statistics.median(ts)
    return {
        "value": round(med * 1e6, 1), "unit": "us", "cores": threads, "kind": "port",
        "sample": f"median of {n} full calls after 1 warm-up of the torch CPU path on the same "
                  f"{case['name']} tensors (unpack+gather+dequant+fp16 matmul per call)",
        "weight_GBps": round(case["wbytes"] / med * 1e-9, 3),
    }


def run_transposed(args, dev):
    """``--transposed``: the gradient for x of the workload's layer, gx[M, K] = gy[M, N] @ W^T
    (gptq_hip_gemm_tiled_transposed on the transposed tiled copy), timed like a forward step and checked against
    the oracle's dequantised weight.  One JSON line; no secondary records."""
    from autogptq.tvm_amd import _lib, ops
    from autogptq.tvm_amd.pack import synth_layer
    from oracle import c_oracle

    bits, K, N, gs, desc_act, M = WORKLOADS[args.workload]
    L = synth_layer(2000 + sorted(WORKLOADS).index(args.workload), K, N, bits, gs, desc_act, M=1)
    qz, sc = L["qzeros"].to(dev), L["scales"].to(dev)
    g = L["g_idx"].to(dev) if desc_act else None
    wbytes = K * N * bits // 8
    copies = max(2, -(-2 * INFINITY_CACHE_BYTES // wbytes))
    gen = torch.Generator().manual_seed(99)
    xsrc, qts, szt = None, [], None
    for c in range(copies):
        q = L["qweight"].to(dev) if c == 0 else torch.randint(
            -(1 << 31), (1 << 31) - 1, L["qweight"].shape, generator=gen, dtype=torch.int64).to(torch.int32).to(dev)
        if c == 0 and desc_act:
            xsrc = ops.tile_prepare(q, qz, sc, g, bits, gs)[2]
        qt, t = ops.tile_prepare_transposed(q, qz, sc, xsrc, bits, gs)
        qts.append(qt)
        szt = t if c == 0 else szt
    gy_cpu = torch.randn(M, N, generator=torch.Generator().manual_seed(7)).half()
    gy, gx = gy_cpu.to(dev), torch.empty((M, K), dtype=torch.float16, device=dev)
    plan = _lib.select_tiled_transposed(M, K, N, bits, gs)
    ws = torch.zeros(max(plan.workspace_bytes, 16), dtype=torch.uint8, device=dev)
    lib = _lib.lib()
    vp = ctypes.c_void_p
    ptr = lambda t: vp(t.data_ptr()) if t is not None else None
    qps = [ptr(q) for q in qts]
    a_gy, a_szt, a_xsrc, a_gx, a_ws = ptr(gy), ptr(szt), ptr(xsrc), ptr(gx), ptr(ws)
    planp = ctypes.byref(plan)

    def step(i, stream):
        rc = lib.gptq_hip_gemm_tiled_transposed(a_gy, qps[i % copies], a_szt, a_xsrc, a_gx, a_ws, ws.numel(), M, K, N, bits,
                                                gs, planp, stream)
        if rc != 0:
            raise RuntimeError(f"gptq_hip_gemm_tiled_transposed failed: {_lib.strerror(rc)}")

    step(0, vp(torch.cuda.current_stream(dev).cuda_stream))
    torch.cuda.synchronize(dev)
    w16 = torch.from_numpy(c_oracle.dequant(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(),
                                            L["g_idx"].numpy(), bits).copy())
    want = gy_cpu.float() @ w16.float().t()
    err = (gx.float().cpu() - want).abs()
    ok = bool((err <= 1e-2 + 1e-2 * want.abs()).all())
    stream = torch.cuda.Stream(device=dev)
    with torch.cuda.stream(stream):
        sp = vp(stream.cuda_stream)
        for i in range(args.warmup):
            step(i, sp)
        stream.synchronize()
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr, stream=stream):
        spg = vp(torch.cuda.current_stream(dev).cuda_stream)
        for i in range(args.steps):
            step(args.warmup + i, spg)
    gr.replay()
    torch.cuda.synchronize(dev)
    times = []
    for _ in range(3):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize(dev)
        scrub_cache(dev)   # (the replay is queued behind the scrub, see time_case)
        e0.record()
        gr.replay()
        e1.record()
        torch.cuda.synchronize(dev)
        times.append(e0.elapsed_time(e1) * 1e3 / args.steps)
    us = min(times)
    tflops = 2 * M * K * N / us * 1e-6
    print(json.dumps({
        "metric": f"transposed GEMM latency (gradient for x), int{bits} {K}x{N} M={M}", "value": round(us, 3), "unit": "us",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(us * 1e-3, 6),
        "higher_is_better": False, "scaling": "weak", "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": args.workload + " (transposed)", "bits": bits, "K": K, "N": N, "M": M, "group_size": gs,
                   "desc_act": desc_act, "weight_copies": copies, "entry": "gptq_hip_gemm_tiled_transposed",
                   "plan": {k: v for k, v in plan.as_dict().items()
                            if k in ("kernel", "row_tiles", "waves_n", "waves_k", "split_k", "grid_x", "grid_y", "grid_z")}},
        "parity": {"ok": ok, "max_abs_err": round(float(err.max()), 6), "rtol": 1e-2, "atol": 1e-2},
        "tflops": round(tflops, 2),
        "roofline": {"bound": "mfma", "achieved": round(tflops, 2), "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(tflops / MFMA_FP16_PEAK_TFLOPS, 4), "traffic": None},
    }))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default=DEFAULT_WORKLOAD, choices=sorted(WORKLOADS))
    ap.add_argument("--sweep", action="store_true", help="also time every workload in WORKLOADS")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-secondary", action="store_true", help="default workload only: skip the secondary records")
    ap.add_argument("--unprepared", action="store_true",
                    help="decode on activation-order layers: time gptq_hip_gemm on the checkpoint's tensors "
                         "instead of gptq_hip_gemm_sorted on the load-time prepared ones")
    ap.add_argument("--prepared", default="auto", choices=("auto", "none", "sorted", "tiled"),
                    help="which copy of the layer to run on: the module's own choice (auto), the checkpoint's "
                         "tensors, the sorted copy or the tiled copy")
    ap.add_argument("--kernel", type=int, default=0, help="force a kernel family (1 gather, 2 grouped, 3 blocked)")
    ap.add_argument("--split-k", type=int, default=0, help="force the split-K factor")
    ap.add_argument("--waves-n", type=int, default=0, help="force the waves per workgroup along N (STREAM kernel: along K)")
    ap.add_argument("--transposed", action="store_true",
                    help="time the gradient for x of the workload's layer (gy[M, N] @ W^T on the transposed tiled "
                         "copy) instead of the forward product")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="only run a plain 256 MiB device copy a few times (known traffic, for scaling the "
                         "FETCH_SIZE / WRITE_SIZE counters of a profiler run) and exit")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures the QuantLinear kernels on ONE GPU; --gpus must be 1 "
              "(the path shards by output columns with no exchange between GPUs)", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the kernels have no CPU fallback", file=sys.stderr)
        sys.exit(3)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        nbytes = 256 << 20
        src = torch.arange(nbytes // 4, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize(dev)
        print(json.dumps({"copy_calibration": {"bytes_read": nbytes, "bytes_written": nbytes, "launches": 5,
                                               "kernel": "torch elementwise copy (int32)"}}))
        return
    if args.transposed:
        run_transposed(args, dev)
        return
    forced = bool(args.kernel or args.split_k or args.waves_n)
    prepared = None if (args.unprepared or forced) else prepared_mode(args.workload)
    if args.prepared != "auto" and not forced:
        prepared = None if args.prepared == "none" else args.prepared
    case = build_case(args.workload, dev, args.kernel, args.split_k, args.waves_n, prepared=prepared)
    ok, max_err = check_case(case, dev)
    torch.cuda.synchronize(dev)
    t = time_case(case, dev, args.steps, args.warmup)
    torch.cuda.synchronize(dev)
    s = summarize(case, t)
    if prepared and plain_applies(args.workload):
        plain = build_case(args.workload, dev)
        okp, _ = check_case(plain, dev)
        s["unprepared_us"] = round(time_case(plain, dev, min(args.steps, 100), min(args.warmup, 10))["us"], 3)
        ok = ok and okp
        del plain
        torch.cuda.empty_cache()
    bits, K, N, gs, desc_act, M = WORKLOADS[args.workload]
    gemv = M <= 8
    line = {
        "metric": f"GEMV latency, int{bits} {K}x{N} M={M}, cache-cold" if gemv
                  else f"GEMM latency, int{bits} {K}x{N} M={M}",
        "value": s["us"], "unit": "us", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(s["us"] * 1e-3, 6), "higher_is_better": False, "scaling": "weak",
        "vs_baseline": None, "dtype": "f16", "data": "synthetic",
        "config": {"workload": args.workload, "bits": bits, "K": K, "N": N, "M": M, "group_size": gs,
                   "desc_act": desc_act, "weight_copies": len(case["qweights"]), "plan": s["plan"],
                   "entry": ENTRY[prepared], "prepared": PREPARED_NOTE[prepared]},
        "parity": {"ok": ok, "max_abs_err": round(max_err, 6), "rtol": 1e-2, "atol": 1e-2},
        "timing": {k: s[k] for k in ("eager_us", "graph_us", "graph_error", "unprepared_us") if k in s},
        "hbm_frac": s["hbm_frac"], "tflops": s["TFLOPs"],
    }
    line["roofline"] = roofline_of(args.workload, s)
    if args.workload == DEFAULT_WORKLOAD and not forced and not args.unprepared and not args.no_secondary:
        # the other halves of the metric, each a timed record of its own with its roofline and parity
        secondary = []
        for name in SECONDARY_WORKLOADS:
            prep = prepared_mode(name)
            c = build_case(name, dev, prepared=prep)
            okc, errc = check_case(c, dev)
            r = summarize(c, time_case(c, dev, args.steps, args.warmup))
            secondary.append({
                "workload": name, "value": r["us"], "unit": "us", "steps": args.steps, "warmup": args.warmup,
                "timing": {k: r[k] for k in ("eager_us", "graph_us", "graph_error") if k in r},
                "entry": ENTRY[prep], "prepared": PREPARED_NOTE[prep], "plan": r["plan"],
                "hbm_frac": r["hbm_frac"], "tflops": r["TFLOPs"], "mfma_frac": r["mfma_frac"],
                "roofline": roofline_of(name, r),
                "parity": {"ok": okc, "max_abs_err": round(errc, 6), "rtol": 1e-2, "atol": 1e-2},
            })
            del c
            torch.cuda.empty_cache()
        line["secondary"] = secondary
    if args.sweep:
        sweep = []
        for name, prep in [(n, pr) for n in sorted(WORKLOADS) for pr in (None, "sorted", "tiled")]:
            if ((prep is None and not plain_applies(name)) or (prep == "sorted" and not sorted_applies(name))
                    or (prep == "tiled" and not tiled_applies(name))):
                continue
            c = build_case(name, dev, prepared=prep)
            okc, errc = check_case(c, dev)
            r = summarize(c, time_case(c, dev, min(args.steps, 100), min(args.warmup, 10)))
            r["prepared"] = prep
            r["module_choice"] = prep == prepared_mode(name)
            r["parity_ok"] = okc
            r["max_abs_err"] = round(errc, 6)
            sweep.append(r)
            del c
            torch.cuda.empty_cache()
        line["sweep"] = sweep
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(case)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
