#!/usr/bin/env python3
"""Benchmark of the GPTQ QuantLinear hot path on one MI355X.

Default workload: the headline configuration of the reference's benchmarks -- 3-bit GEMV, M=1, K=4096, N=11008, group_size=128,
desc_act=True (g_idx from a random permutation), synthetic seeded tensors.  One "step" is one call of the C-ABI
entry point that ``gptq_hip_select_route`` names for the shape (the decision ``QuantLinear.forward`` follows), on
tensors already resident in HBM: ``gptq_hip_gemm_tiled`` on the layer's copy in the tiled format,
``gptq_hip_gemm_sorted`` on its channel-sorted copy, or ``gptq_hip_gemm_plan`` on the checkpoint's own tensors
(``--prepared`` forces a copy; the default run reports the checkpoint-tensor figure too, under
``timing.unprepared_us``).  Steps rotate over enough distinct weight copies to exceed twice the 256 MB Infinity
Cache, so every step streams its packed weights from HBM (cache-cold).

Timing: K steps, and 2 K steps, are captured once each into a HIP graph and replayed inside an event-bracketed
region that sits behind a read of 512 MB (cache scrub), the W warm-up steps and max(K, 256) more untimed steps (a
graph of its own), all queued back to back.  A replay carries a fixed ~10 us of start-up on the GPU whatever sits in
front of it (t(K) = 9.6 us + 6.80 us * K fitted K = 5 ... 1000 on the headline), which at K = 20 would read as
0.5 us per step; a decode loop replays hundreds of kernels per graph, so the figure reported is the time of K
steps with that constant taken out: t(2 K) - t(K).  Five regions of each; ``value`` is the median of the
differences, ``timing.min_us`` their minimum, ``timing.region_us`` the plain t(K) / K and
``timing.replay_overhead_us`` the constant, 2 t(K) - t(2 K).

Prints ONE JSON line (see the keys below).  ``roofline.achieved`` is algorithmic bytes (packed qweight only,
K*N*bits/8) or flops (2*M*K*N) per launch divided by the median step time measured here with HIP events on the
launch stream.  ``secondary`` holds one record like it for every other point of the configurations the metric is
quoted on (configs[0], the 4-bit twin of the headline, the decode sweep, the prefill sweep, the one-group 3-bit
layers), each with its own roofline and parity check.  ``cpu_baseline`` times the CPU oracle (the restatement of
the reference's torch path) on this box's host cores: all cores, one core, and the matmul alone on a
pre-dequantised weight.

Other workloads: ``--workload NAME`` (see WORKLOADS), ``--sweep`` adds a table of every workload on every copy
of the layer under "sweep" in the same JSON line.
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
    # prompts on a narrow layer (the attention projections of a 4096-wide block): shorter row blocks, no K ranges
    "int4-4096x4096-act-m64": (4, 4096, 4096, 128, True, 64),
    "int4-4096x4096-act-m128": (4, 4096, 4096, 128, True, 128),
    "int3-4096x4096-act-m128": (3, 4096, 4096, 128, True, 128),
    "int4-4096x4096-act-m256": (4, 4096, 4096, 128, True, 256),
    # a long, narrow layer at prompt sizes: K in three ranges, two turns of the chip
    "int3-36864x9216-g1-m128": (3, 36864, 9216, -1, True, 128),
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
# every point of the configurations the metric is quoted on
for _K, _N in ((4096, 4096), (4096, 11008), (11008, 4096)):
    for _M in (1, 2, 4, 8):
        WORKLOADS.setdefault(f"c3-int4-{_K}x{_N}-m{_M}", (4, _K, _N, 128, False, _M))
for _K, _N in ((4096, 11008), (11008, 4096)):
    for _b in (4, 3):
        for _M in (16, 64, 128, 256):
            WORKLOADS.setdefault(f"c4-int{_b}-{_K}x{_N}-act-m{_M}", (_b, _K, _N, 128, True, _M))
for _K, _N in ((9216, 9216), (9216, 36864), (36864, 9216)):
    for _M in (1, 32):
        WORKLOADS.setdefault(f"c5-int3-{_K}x{_N}-g1-m{_M}", (3, _K, _N, -1, True, _M))
DEFAULT_WORKLOAD = "c2-int3-4096x11008-act-m1"
# timed in the default run next to the headline, each as a record of its own: configs[0], the headline's 4-bit twin,
# and every point of the decode sweep (configs[2]), the prefill sweep (configs[3]) and the one-group layers (configs[4])
SECONDARY_WORKLOADS = tuple(
    ["c1-int4-4096x4096-m1", "int4-4096x11008-act-m1"]
    + [f"c3-int4-{k}x{n}-m{m}" for k, n in ((4096, 4096), (4096, 11008), (11008, 4096)) for m in (1, 2, 4, 8)]
    + [f"c4-int{b}-{k}x{n}-act-m{m}" for k, n in ((4096, 11008), (11008, 4096)) for b in (4, 3) for m in (16, 64, 128, 256)]
    + [f"c5-int3-{k}x{n}-g1-m{m}" for k, n in ((9216, 9216), (9216, 36864), (36864, 9216)) for m in (1, 32)])

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


class Layer:
    """One synthetic layer (bits, K, N, group_size, desc_act) shared by every workload on it: the seeded tensors on
    the CPU, the oracle's dequantised weight, and per copy format ("tiled", "sorted", None = the checkpoint's own
    tensors) enough distinct weight copies on the device to exceed twice the Infinity Cache."""

    def __init__(self, key, dev, max_rows: int):
        from autogptq.tvm_amd.pack import synth_layer

        self.key = key
        bits, K, N, gs, desc_act = key
        self.dev = dev
        self.L = synth_layer(2000 + (bits * 131 + K * 7 + N * 3 + (1 if desc_act else 0) + (gs & 0xff)) % 9973, K, N, bits,
                             gs, desc_act, M=max_rows)
        self.rows = max_rows
        self.wbytes = K * N * bits // 8
        self.copies = max(2, -(-2 * INFINITY_CACHE_BYTES // self.wbytes), int(os.environ.get("GPTQ_BENCH_MIN_COPIES", "0")))
        self.qzeros, self.scales = self.L["qzeros"].to(dev), self.L["scales"].to(dev)
        # a layer of one group has no order of groups to follow: its g_idx is all zeros, QuantLinear passes none
        # to the kernels (and no channel maps of the tiled copy), and neither does this harness
        self.mapped = bool(desc_act and 0 < gs < K)
        self.g_idx = self.L["g_idx"].to(dev) if self.mapped else None
        self.x = self.L["x"].to(dev)
        self._fmt = {}
        self._want = None

    def raw_copy(self, c: int):
        """Copy 0 is the seeded layer; the others are distinct random packed words (every int32 pattern is a valid
        block of codes), drawn on the device."""
        if c == 0:
            return self.L["qweight"].to(self.dev)
        gen = torch.Generator(device=self.dev).manual_seed(99 + c)
        return torch.randint(-(1 << 31), (1 << 31) - 1, tuple(self.L["qweight"].shape), generator=gen, dtype=torch.int64,
                             device=self.dev).to(torch.int32)

    def fmt(self, prepared):
        """{"qweights": [...], "aux": [per copy tuple], "kmap": ...} for a copy format, built once."""
        from autogptq.tvm_amd import ops
        from autogptq.tvm_amd.pack import sort_channels_by_group

        if prepared in self._fmt:
            return self._fmt[prepared]
        bits, K, N, gs, desc_act = self.key
        out = {"qweights": [], "aux": [], "kmap": None}
        for c in range(self.copies):
            q = self.raw_copy(c)
            if prepared == "tiled":
                # (every copy brings its own scale / zero words and channel maps, as every layer of a model does)
                qtile, sz, xsrc, kinv = ops.tile_prepare(q, self.qzeros, self.scales, self.g_idx, bits, gs)
                out["aux"].append((sz, xsrc if self.mapped else None, kinv if self.mapped else None))
                q = qtile
            out["qweights"].append(q)
        if prepared == "sorted":
            out["qweights"][0], out["kmap"] = sort_channels_by_group(out["qweights"][0], self.g_idx, bits, gs)
        if prepared != "tiled":
            # the layer's other tensors, one set per copy as well (qzeros, scales, and g_idx or the sorted copy's map)
            g_or_map = out["kmap"] if out["kmap"] is not None else self.g_idx
            out["aux"] = [(self.qzeros, self.scales, g_or_map)] + [
                (self.qzeros.clone(), self.scales.clone(), g_or_map.clone() if g_or_map is not None else None)
                for _ in range(self.copies - 1)]
        self._fmt[prepared] = out
        return out

    def drop(self, prepared):
        self._fmt.pop(prepared, None)
        torch.cuda.empty_cache()

    def want(self):
        """x @ W in fp32 on the oracle's dequantised weight, for all rows of x."""
        from oracle import c_oracle

        if self._want is None:
            L = self.L
            w16 = torch.from_numpy(c_oracle.dequant(L["qweight"].numpy(), L["qzeros"].numpy(), L["scales"].numpy(),
                                                    L["g_idx"].numpy(), self.key[0]).copy())
            self._want = L["x"].float() @ w16.float()
        return self._want


_layers = {}


def layer_of(name: str, dev, max_rows: int = 0) -> Layer:
    """The layer of a workload, kept for the other workloads on it (one layer at a time: a new one frees the last)."""
    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    key = (bits, K, N, gs, desc_act)
    rows = max(M, max_rows)
    lay = _layers.get(key)
    if lay is None or lay.rows < rows:
        _layers.clear()
        torch.cuda.empty_cache()
        lay = _layers[key] = Layer(key, dev, rows)
    return lay


def build_case(name: str, dev, kernel: int = 0, split_k: int = 0, waves_n: int = 0, prepared=None, max_rows: int = 0):
    """prepared: the copy of the layer the step runs on: "sorted" (channels of an activation-order layer sorted by
    group, gptq_hip_gemm_sorted), "tiled" (the tiled format, gptq_hip_gemm_tiled), or None (the checkpoint's
    tensors, gptq_hip_gemm_plan); prepared_mode(name) is the library's own choice."""
    from autogptq.tvm_amd import _lib, ops

    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    lay = layer_of(name, dev, max_rows)
    f = lay.fmt(prepared)
    case = {
        "name": name, "bits": bits, "K": K, "N": N, "gs": gs, "desc_act": desc_act, "M": M, "layer": lay,
        "x": lay.x[:M], "y": torch.empty((M, N), dtype=torch.float16, device=dev),
        "wbytes": lay.wbytes, "flops": 2 * M * K * N, "kmap": f["kmap"], "prepared": prepared,
        "qweights": f["qweights"], "aux": f["aux"],
    }
    act = lay.mapped and prepared != "sorted"   # the sorted copy is planned like contiguous groups
    if prepared == "tiled":
        plan = _lib.select_tiled(M, K, N, bits, gs)
    elif prepared == "sorted" and not (kernel or split_k or waves_n):
        plan = ops.sorted_plan(M, K, N, bits, gs)
    elif kernel or split_k or waves_n:
        if not kernel:
            kernel = _lib.select(M, K, N, bits, gs, act).kernel
        plan = _lib.plan_for(kernel, M, K, N, bits, gs, act, split_k, waves_n)
    else:
        plan = _lib.select(M, K, N, bits, gs, act)
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
    """The copy of the layer gptq_hip_select_route names for this workload when all three are on offer (the
    decision QuantLinear.forward follows), or None for the checkpoint's own tensors."""
    from autogptq.tvm_amd import _lib

    bits, K, N, gs, desc_act, M = WORKLOADS[name]
    r = _lib.select_route(M, K, N, bits, gs, desc_act, switch_rows=(0, 0, 0))
    return {_lib.ROUTE_TILED: "tiled", _lib.ROUTE_SORTED: "sorted"}.get(r.copy)


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
        aux = [tuple(ptr(t) for t in c) for c in case["aux"]]

        def step(i, stream):
            sz, xsrc, kinv = aux[i % n]
            rc = lib.gptq_hip_gemm_tiled(x, qws[i % n], sz, xsrc, kinv, None, y, ws, wsb, M, K, N, bits, gs, planp, stream)
            if rc != 0:
                raise RuntimeError(f"gptq_hip_gemm_tiled failed: {_lib.strerror(rc)}")

        return step
    fn = lib.gptq_hip_gemm_sorted if case["kmap"] is not None else lib.gptq_hip_gemm_plan
    aux = [tuple(ptr(t) for t in c) for c in case["aux"]]

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


REGIONS = 5
PRE_STEPS = 256   # untimed steps queued in front of the timed graph: enough GPU work (a millisecond and more) for the
                  # host to have submitted the timed graph before the GPU gets to it


def time_case(case, dev, steps: int, warmup: int, eager: bool = False):
    """Duration of one step in microseconds.  K steps, and 2 K steps, are captured once each into a HIP graph and
    replayed inside an event-bracketed region; in front of it, queued back to back on the same stream: a read of
    512 MB (cache scrub), the W warm-up steps and max(K, PRE_STEPS) more untimed steps, each a graph of its own, so
    that the timed steps start on a busy GPU (the first steps behind an idle or scrubbed GPU take ~2 us longer
    each) and the host is far ahead of the GPU.  A replay still costs the GPU a fixed ~10 us at its start, which
    would make the figure depend on K (20 steps: +0.5 us each); ``us`` is therefore the time of K steps with that
    constant taken out, (t(2 K) - t(K)) / K: the median over REGIONS pairs of regions, ``min_us`` their minimum.
    ``region_us`` = t(K) / K as it stands, ``replay_overhead_us`` = 2 t(K) - t(2 K).  The weight copy of step i is
    i mod copies over warm-up, untimed and timed steps alike, and copies * bytes is at least twice the Infinity
    Cache, so no timed step finds its weights cached.  ``eager_us`` (on request) = the same K steps launched one
    by one."""
    step = make_step(case, dev)
    stream = torch.cuda.Stream(device=dev)
    res = {}
    with torch.cuda.stream(stream):
        sp = ctypes.c_void_p(stream.cuda_stream)
        for i in range(max(warmup, 2)):       # (first calls: lazy initialisation of the runtime for these kernels)
            step(i, sp)
        stream.synchronize()
        if eager:
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
    try:
        graphs = []
        pre = max(steps, PRE_STEPS)
        for first, count in ((0, warmup), (warmup, pre), (warmup + pre, steps), (warmup + pre, 2 * steps)):
            g = torch.cuda.CUDAGraph()
            if count > 0:
                with torch.cuda.graph(g, stream=stream):
                    spg = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
                    for i in range(count):
                        step(first + i, spg)
            graphs.append(g if count > 0 else None)
        g_warm, g_pre, g_k, g_2k = graphs
        g_pre.replay()
        g_k.replay()
        g_2k.replay()
        torch.cuda.synchronize(dev)

        def region(g):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize(dev)
            scrub_cache(dev)
            if g_warm is not None:
                g_warm.replay()
            g_pre.replay()
            e0.record()
            g.replay()
            e1.record()
            torch.cuda.synchronize(dev)
            return e0.elapsed_time(e1) * 1e3

        t_k = [region(g_k) for _ in range(REGIONS)]
        t_2k = [region(g_2k) for _ in range(REGIONS)]
        slopes = sorted((b - a) / steps for a, b in zip(sorted(t_k), sorted(t_2k)))
        res["graph_us"] = statistics.median(slopes)
        res["min_us"] = slopes[0]
        res["region_us"] = statistics.median(t_k) / steps              # one replay of K steps, its start-up included
        res["replay_overhead_us"] = max(0.0, 2 * statistics.median(t_k) - statistics.median(t_2k))
    except Exception as exc:  # graph capture unavailable: report the eager figure only
        res["graph_error"] = repr(exc)[:200]
        if "eager_us" not in res:
            return time_case(case, dev, steps, warmup, eager=True) | {"graph_error": res["graph_error"]}
    res["us"] = res.get("graph_us", res.get("eager_us"))
    return res


def check_case(case, dev):
    """The timed path's output against the oracle, for the first weight copy."""
    step = make_step(case, dev)
    step(0, ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    torch.cuda.synchronize(dev)
    want = case["layer"].want()[:case["M"]]
    got = case["y"].float().cpu()
    err = (got - want).abs()
    ok = bool((err <= 1e-2 + 1e-2 * want.abs()).all())
    return ok, float(err.max())


def summarize(case, t):
    us = t["us"]
    out = {"workload": case["name"], "us": round(us, 3)}
    out.update({k: (round(v, 3) if isinstance(v, float) else v) for k, v in t.items() if k not in ("us", "min_us")})
    if "min_us" in t:
        out["min_us"] = round(t["min_us"], 3)
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


def _timed_calls(fn, warmups: int, budget_s: float, most: int = 10):
    for _ in range(warmups):
        fn()
    t0 = time.perf_counter()
    fn()
    first = time.perf_counter() - t0
    n = max(2, min(most - 1, int(budget_s / max(first, 1e-4)) - 1))
    ts = [first]
    for _ in range(n):
        t0 = time.perf_counter()
        fn()
        ts.append(time.perf_counter() - t0)
    return statistics.median(ts), len(ts)


def cpu_baseline(case, budget_s: float = 10.0):
    """The reference's CPU path (oracle restatement of qlinear.py:198-245: unpack + gather + dequant + fp16 matmul
    on every call) on this box's host cores: with all of them, with one, and the matmul alone on a weight that was
    dequantised beforehand (what remains of a call when the unpack and dequant steps are taken out)."""
    from oracle import gptq_oracle as orc

    L = case["layer"].L
    M = case["M"]
    x = L["x"][:M]
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "0") or 0) or (os.cpu_count() or 1))
    args = (x, L["qweight"], L["qzeros"], L["scales"], L["g_idx"], None, case["bits"])
    torch.set_num_threads(threads)
    med, n = _timed_calls(lambda: orc.forward_ref(*args), 3, budget_s)
    w16 = orc.dequant_ref(L["qweight"], L["qzeros"], L["scales"], L["g_idx"], case["bits"])
    mm, n_mm = _timed_calls(lambda: orc.matmul_only_ref(x, w16), 3, 2.0)
    torch.set_num_threads(1)
    one, n_one = _timed_calls(lambda: orc.forward_ref(*args), 1, budget_s, most=5)
    torch.set_num_threads(threads)
    return {
        "value": round(med * 1e6, 1), "unit": "us", "cores": threads, "kind": "port",
        "sample": f"median of {n} full calls after 3 warm-ups of the torch CPU path on the same {case['name']} "
                  f"tensors (unpack+gather+dequant+fp16 matmul per call), {threads} threads",
        "weight_GBps": round(case["wbytes"] / med * 1e-9, 3),
        "single_thread": {"value": round(one * 1e6, 1), "unit": "us", "cores": 1,
                          "sample": f"median of {n_one} full calls after 1 warm-up, torch.set_num_threads(1)"},
        "matmul_only": {"value": round(mm * 1e6, 1), "unit": "us", "cores": threads,
                        "sample": f"median of {n_mm} calls of x.half() @ W on the pre-dequantised fp16 weight "
                                  f"after 3 warm-ups"},
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


def _slope_us(launch, dev, n: int, regions: int = 5) -> float:
    """Microseconds per launch of a chain of dependent launches, as the difference of a graph of 2 n launches and
    one of n (median over `regions` pairs), so that the fixed start-up of a replay cancels."""
    def graph(count):
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for j in range(count):
                launch(j)
        return g
    launch(0)
    torch.cuda.synchronize(dev)
    g1, g2 = graph(n), graph(2 * n)
    out = []
    for _ in range(regions + 1):
        t = []
        for g in (g1, g2):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize(dev)
            a.record()
            g.replay()
            b.record()
            torch.cuda.synchronize(dev)
            t.append(a.elapsed_time(b) * 1e3)
        out.append((t[1] - t[0]) / n)
    return float(statistics.median(out[1:]))


def run_machine(args, dev):
    """What this GPU gives the product kernels, measured with the library's probe kernels: the cost of a launch in a
    chain of launches, the cost of a plain read of a layer's bytes by as many workgroups as the decode kernels use
    (every launch a region that no cache still holds), and the rate of loads that hit L2 while the same CU also
    streams from HBM (what the activation fragments of a matmul kernel pay next to its weight stream)."""
    import numpy as np
    from autogptq.tvm_amd import _lib
    l = _lib.lib()
    def cur():      # (inside a capture the current stream is the capturing one)
        return ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)

    sink = torch.zeros(4, dtype=torch.int32, device=dev)
    big = torch.empty(1 << 30, dtype=torch.uint8, device=dev)
    big.view(torch.int32).random_(0, 1 << 30)
    hot = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    hot.view(torch.int32).random_(0, 1 << 30)
    ticks = torch.zeros(4 * 256, dtype=torch.int64, device=dev)

    def check(rc):
        if rc != 0:
            raise RuntimeError(f"gptq_hip_probe: {rc}")

    out = {"launch_us": {}, "stream_read": [], "l2_hit_loads_per_cu": {}}
    for wgs in (256, 432, 1024):
        out["launch_us"][str(wgs)] = round(_slope_us(
            lambda j: check(l.gptq_hip_probe(_lib.PROBE_EMPTY, None, 0, None, 0, wgs, 0, 0, 0, None, None, cur())),
            dev, args.steps), 3)
    for label, nbytes in (("int3 4096x11008", 4096 * 11008 * 3 // 8), ("int3 9216x36864", 9216 * 36864 * 3 // 8)):
        nbytes = nbytes // 4096 * 4096
        regions = big.numel() // nbytes
        for wgs in (256, 432, 1024, 2048):
            us = _slope_us(
                lambda j: check(l.gptq_hip_probe(_lib.PROBE_STREAM, ctypes.c_void_p(big.data_ptr() + (j % regions) * nbytes),
                                                 nbytes, None, 0, wgs, 0, 0, 0, None,
                                                 ctypes.c_void_p(sink.data_ptr()), cur())),
                dev, max(regions, min(args.steps, 2 * regions)))
            out["stream_read"].append({"bytes_of": label, "bytes": nbytes, "workgroups": wgs, "us": round(us, 3),
                                       "GBps": round(nbytes / us * 1e-3, 1)})
    iters, wall_hz = 400, 1e8     # the wall clock of this GPU ticks at 100 MHz
    per_cu = 2 * iters * 8 * 1024
    for label, mode, depth in (("alone", 0, 1), ("next to two more such waves", 1, 1),
                               ("next to an HBM stream, 1 request per round and wave", 2, 1),
                               ("next to an HBM stream, 4 requests per round and wave", 2, 4),
                               ("next to an HBM stream, 8 requests per round and wave", 2, 8)):
        rates = []
        for _ in range(3):
            ticks.zero_()
            check(l.gptq_hip_probe(_lib.PROBE_MIXED, ctypes.c_void_p(big.data_ptr()), big.numel(),
                                   ctypes.c_void_p(hot.data_ptr()), hot.numel(), 256, iters, mode, depth,
                                   ctypes.c_void_p(ticks.data_ptr()), ctypes.c_void_p(sink.data_ptr()), cur()))
            torch.cuda.synchronize(dev)
            tk = ticks.view(256, 4)[:, :2].double().max(dim=1).values      # the slower of a CU's two reading waves
            rates.append(float((per_cu / (tk / wall_hz)).median()) * 1e-9)
        out["l2_hit_loads_per_cu"][label] = {"GBps": round(float(np.median(rates)), 1)}
    out["note"] = ("launch_us and stream_read: per launch of a chain of dependent launches, graph of 2 n minus graph of "
                   "n; stream_read regions rotate through 1 GiB so that no cache holds them; l2_hit_loads_per_cu: two "
                   "waves of a 256-thread workgroup (one workgroup per CU) read a 1 MiB buffer with direct loads into LDS, 16 B "
                   "per lane, a round of eight 1 KiB requests in flight behind the round waited for; median over the "
                   "256 workgroups")
    print(json.dumps({"machine": out}))


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
    ap.add_argument("--kernel", type=int, default=0, help="force a kernel family (2 grouped, 3 stream)")
    ap.add_argument("--split-k", type=int, default=0, help="force the split-K factor")
    ap.add_argument("--waves-n", type=int, default=0, help="force the waves per workgroup along N (STREAM kernel: along K)")
    ap.add_argument("--transposed", action="store_true",
                    help="time the gradient for x of the workload's layer (gy[M, N] @ W^T on the transposed tiled "
                         "copy) instead of the forward product")
    ap.add_argument("--machine", action="store_true",
                    help="only measure what the GPU gives the kernels (launch cost, plain streaming reads by as many "
                         "workgroups, L2-hit loads next to an HBM stream in one CU) with the library's probe kernels")
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
    if args.machine:
        run_machine(args, dev)
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
    t = time_case(case, dev, args.steps, args.warmup, eager=True)
    torch.cuda.synchronize(dev)
    s = summarize(case, t)
    if prepared and plain_applies(args.workload):
        plain = build_case(args.workload, dev)
        okp, _ = check_case(plain, dev)
        s["unprepared_us"] = round(time_case(plain, dev, min(args.steps, 100), min(args.warmup, 10))["us"], 3)
        ok = ok and okp
        del plain
        case["layer"].drop(None)
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
        "timing": {"statistic": f"median over {REGIONS} pairs of timed regions of t(2 K) - t(K), K = {args.steps} steps "
                                f"(graph replay; the fixed start-up of a replay cancels)",
                   **{k: s[k] for k in ("min_us", "region_us", "replay_overhead_us", "eager_us", "graph_us",
                                        "graph_error", "unprepared_us") if k in s}},
        "hbm_frac": s["hbm_frac"], "tflops": s["TFLOPs"],
    }
    line["roofline"] = roofline_of(args.workload, s)
    cpu = None
    if not args.no_cpu_baseline:
        cpu = cpu_baseline(case)      # (while the headline's layer is still the one held)
    if args.workload == DEFAULT_WORKLOAD and not forced and not args.unprepared and not args.no_secondary:
        # the other points of the metric's configurations, each a timed record of its own with its roofline and
        # parity; workloads on one layer follow each other so that the layer is built once
        seen = {WORKLOADS[args.workload]}
        todo = []
        for name in SECONDARY_WORKLOADS:
            if WORKLOADS[name] not in seen:
                seen.add(WORKLOADS[name])
                todo.append(name)
        rows_of = {}
        for name in todo:
            rows_of[WORKLOADS[name][:5]] = max(rows_of.get(WORKLOADS[name][:5], 0), WORKLOADS[name][5])
        todo.sort(key=lambda n: (list(rows_of).index(WORKLOADS[n][:5]), WORKLOADS[n][5]))
        secondary = []
        for name in todo:
            prep = prepared_mode(name)
            c = build_case(name, dev, prepared=prep, max_rows=rows_of[WORKLOADS[name][:5]])
            okc, errc = check_case(c, dev)
            r = summarize(c, time_case(c, dev, args.steps, args.warmup))
            secondary.append({
                "workload": name, "value": r["us"], "min_us": r.get("min_us"), "unit": "us", "steps": args.steps,
                "warmup": args.warmup, "entry": ENTRY[prep], "plan": r["plan"],
                "hbm_frac": r["hbm_frac"], "tflops": r["TFLOPs"], "mfma_frac": r["mfma_frac"],
                "roofline": roofline_of(name, r),
                "parity": {"ok": okc, "max_abs_err": round(errc, 6), "rtol": 1e-2, "atol": 1e-2},
            })
            del c
        line["secondary"] = secondary
    if args.sweep:
        sweep = []
        names = sorted(WORKLOADS, key=lambda n: (WORKLOADS[n][:5], WORKLOADS[n][5]))
        for name, prep in [(n, pr) for n in names for pr in (None, "sorted", "tiled")]:
            if ((prep is None and not plain_applies(name)) or (prep == "sorted" and not sorted_applies(name))
                    or (prep == "tiled" and not tiled_applies(name))):
                continue
            rows = max(v[5] for v in WORKLOADS.values() if v[:5] == WORKLOADS[name][:5])
            c = build_case(name, dev, prepared=prep, max_rows=rows)
            okc, errc = check_case(c, dev)
            r = summarize(c, time_case(c, dev, min(args.steps, 100), min(args.warmup, 10)))
            r["prepared"] = prep
            r["module_choice"] = prep == prepared_mode(name)
            r["parity_ok"] = okc
            r["max_abs_err"] = round(errc, 6)
            sweep.append(r)
            del c
        line["sweep"] = sweep
    if cpu is not None:
        line["cpu_baseline"] = cpu
    print(json.dumps(line))


if __name__ == "__main__":
    main()
