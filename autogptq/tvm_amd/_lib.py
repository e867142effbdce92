"""ctypes binding of ``csrc/libgptq_hip.so`` (the C ABI declared in include/gptq_hip.h).

The library is the only compute path: if it is missing this module raises, it never
falls back to a CPU or eager implementation.
"""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "csrc", "libgptq_hip.so")

OK = 0
ERR_BAD_ARG = -1
ERR_UNSUPPORTED = -2
ERR_WORKSPACE = -3
ERR_LAUNCH = -4

KERNEL_GROUPED = 2
KERNEL_STREAM = 3
KERNEL_TILED = 4
KERNEL_TILED_DECODE = 5

ABI_SYMBOLS = (
    "gptq_hip_select",
    "gptq_hip_plan_for",
    "gptq_hip_workspace_bytes",
    "gptq_hip_workspace_init",
    "gptq_hip_gemm",
    "gptq_hip_gemm_plan",
    "gptq_hip_gemm_static",
    "gptq_hip_static_workspace_limit",
    "gptq_hip_static_init",
    "gptq_hip_gemm_sorted",
    "gptq_hip_sorted_workspace_bytes",
    "gptq_hip_sort_channels",
    "gptq_hip_tiled_bytes",
    "gptq_hip_tile_prepare",
    "gptq_hip_select_tiled",
    "gptq_hip_select_tiled_decode",
    "gptq_hip_select_route",
    "gptq_hip_tiled_transposed_bytes",
    "gptq_hip_tiled_transposed_table_bytes",
    "gptq_hip_tile_prepare_transposed",
    "gptq_hip_select_tiled_transposed",
    "gptq_hip_gemm_tiled_transposed",
    "gptq_hip_gemm_tiled",
    "gptq_hip_dequant",
    "gptq_hip_probe",
    "gptq_hip_strerror",
    "gptq_hip_abi_version",
    "gptq_hip_build_id",
)
ABI_VERSION = 4


class Plan(ctypes.Structure):
    """Mirror of ``gptq_hip_plan``."""

    _fields_ = [
        ("kernel", ctypes.c_int),
        ("row_tiles", ctypes.c_int),
        ("m_blocks", ctypes.c_int),
        ("waves_n", ctypes.c_int),
        ("waves_k", ctypes.c_int),
        ("split_k", ctypes.c_int),
        ("k_chunk", ctypes.c_int),
        ("grid_x", ctypes.c_int),
        ("grid_y", ctypes.c_int),
        ("grid_z", ctypes.c_int),
        ("block", ctypes.c_int),
        ("lds_bytes", ctypes.c_int),
        ("flags", ctypes.c_int),
        ("workspace_bytes", ctypes.c_size_t),
    ]

    def as_dict(self) -> dict:
        return {name: getattr(self, name) for name, _ in self._fields_}


PLAN_PRIVATE_ZERO_WORKSPACE = 1

COPY_CHECKPOINT, COPY_SORTED, COPY_TILED = 1, 2, 4
ROUTE_CHECKPOINT, ROUTE_SORTED, ROUTE_TILED, ROUTE_LIBRARY = 0, 1, 2, 3
PROBE_EMPTY, PROBE_STREAM, PROBE_MIXED = 0, 1, 2
ROUTE_NAMES = {ROUTE_CHECKPOINT: "plain", ROUTE_SORTED: "sorted", ROUTE_TILED: "tiled", ROUTE_LIBRARY: "library"}


class Route(ctypes.Structure):
    """Mirror of ``gptq_hip_route``."""

    _fields_ = [("copy", ctypes.c_int), ("reserved", ctypes.c_int), ("plan", Plan)]


class GptqHipError(RuntimeError):
    def __init__(self, status: int, where: str):
        self.status = status
        super().__init__(f"{where}: {strerror(status)} (status {status})")


_lib = None


def lib() -> ctypes.CDLL:
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m autogptq.tvm_amd.build` "
            "(there is no fallback path)"
        )
    l = ctypes.CDLL(LIB_PATH)
    vp, i, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    # a library older than the sources beside it is refused before anything else of it is touched
    try:
        l.gptq_hip_abi_version.restype = i
        l.gptq_hip_abi_version.argtypes = []
        l.gptq_hip_build_id.restype = ctypes.c_char_p
        l.gptq_hip_build_id.argtypes = []
        missing = [name for name in ABI_SYMBOLS if not hasattr(l, name)]
    except AttributeError as exc:
        raise RuntimeError(f"{LIB_PATH} is not this package's library ({exc}): rebuild it with "
                           "`python -m autogptq.tvm_amd.build`") from None
    if l.gptq_hip_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{LIB_PATH} has ABI version {l.gptq_hip_abi_version()}, this package expects "
                           f"{ABI_VERSION}: rebuild it with `python -m autogptq.tvm_amd.build`")
    from . import _sources as _build
    built, now = l.gptq_hip_build_id().decode(), _build.source_hash()
    if built != now:
        raise RuntimeError(f"{LIB_PATH} was built from other sources (build id {built}, sources now {now}): "
                           "rebuild it with `python -m autogptq.tvm_amd.build`")
    if missing:
        raise RuntimeError(f"{LIB_PATH} lacks {', '.join(missing)}: rebuild it with `python -m autogptq.tvm_amd.build`")
    l.gptq_hip_select.restype = i
    l.gptq_hip_select.argtypes = [i, i, i, i, i, i, ctypes.POINTER(Plan)]
    l.gptq_hip_plan_for.restype = i
    l.gptq_hip_plan_for.argtypes = [i, i, i, i, i, i, i, i, i, ctypes.POINTER(Plan)]
    l.gptq_hip_workspace_bytes.restype = sz
    l.gptq_hip_workspace_bytes.argtypes = [i, i, i, i, i, i]
    l.gptq_hip_workspace_init.restype = i
    l.gptq_hip_workspace_init.argtypes = [vp, sz, vp]
    l.gptq_hip_gemm.restype = i
    l.gptq_hip_gemm.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, i, vp]
    l.gptq_hip_gemm_plan.restype = i
    l.gptq_hip_gemm_plan.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, i, ctypes.POINTER(Plan), vp]
    l.gptq_hip_gemm_static.restype = i
    l.gptq_hip_gemm_static.argtypes = [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, vp]
    l.gptq_hip_static_init.restype = i
    l.gptq_hip_static_init.argtypes = []
    l.gptq_hip_static_workspace_limit.restype = sz
    l.gptq_hip_static_workspace_limit.argtypes = []
    l.gptq_hip_gemm_sorted.restype = i
    l.gptq_hip_gemm_sorted.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, i, ctypes.POINTER(Plan), vp]
    l.gptq_hip_sorted_workspace_bytes.restype = sz
    l.gptq_hip_sorted_workspace_bytes.argtypes = [i, i, i, i, i]
    l.gptq_hip_sort_channels.restype = i
    l.gptq_hip_sort_channels.argtypes = [vp, vp, vp, vp, i, i, i, i, vp]
    l.gptq_hip_tiled_bytes.restype = sz
    l.gptq_hip_tiled_bytes.argtypes = [i, i, i]
    l.gptq_hip_tile_prepare.restype = i
    l.gptq_hip_tile_prepare.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, vp]
    l.gptq_hip_select_tiled.restype = i
    l.gptq_hip_select_tiled.argtypes = [i, i, i, i, i, ctypes.POINTER(Plan)]
    l.gptq_hip_select_tiled_decode.restype = i
    l.gptq_hip_select_tiled_decode.argtypes = [i, i, i, i, i, ctypes.POINTER(Plan)]
    l.gptq_hip_select_route.restype = i
    l.gptq_hip_select_route.argtypes = [i, i, i, i, i, i, ctypes.c_uint, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(Route)]
    l.gptq_hip_gemm_tiled.restype = i
    l.gptq_hip_gemm_tiled.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, sz, i, i, i, i, i, ctypes.POINTER(Plan), vp]
    l.gptq_hip_tiled_transposed_bytes.restype = sz
    l.gptq_hip_tiled_transposed_bytes.argtypes = [i, i, i]
    l.gptq_hip_tiled_transposed_table_bytes.restype = sz
    l.gptq_hip_tiled_transposed_table_bytes.argtypes = [i, i, i]
    l.gptq_hip_tile_prepare_transposed.restype = i
    l.gptq_hip_tile_prepare_transposed.argtypes = [vp, vp, vp, vp, vp, vp, i, i, i, i, vp]
    l.gptq_hip_select_tiled_transposed.restype = i
    l.gptq_hip_select_tiled_transposed.argtypes = [i, i, i, i, i, ctypes.POINTER(Plan)]
    l.gptq_hip_gemm_tiled_transposed.restype = i
    l.gptq_hip_gemm_tiled_transposed.argtypes = [vp, vp, vp, vp, vp, vp, sz, i, i, i, i, i, ctypes.POINTER(Plan), vp]
    l.gptq_hip_probe.restype = i
    l.gptq_hip_probe.argtypes = [i, vp, sz, vp, sz, i, i, i, i, vp, vp, vp]
    l.gptq_hip_dequant.restype = i
    l.gptq_hip_dequant.argtypes = [vp, vp, vp, vp, vp, i, i, i, i, vp]
    l.gptq_hip_strerror.restype = ctypes.c_char_p
    l.gptq_hip_strerror.argtypes = [i]
    l.gptq_hip_abi_version.restype = i
    l.gptq_hip_abi_version.argtypes = []
    l.gptq_hip_build_id.restype = ctypes.c_char_p
    l.gptq_hip_build_id.argtypes = []
    _lib = l
    return l


def strerror(status: int) -> str:
    return lib().gptq_hip_strerror(int(status)).decode()


def select(M: int, K: int, N: int, bits: int, group_size: int, act_order: bool) -> Plan:
    plan = Plan()
    rc = lib().gptq_hip_select(M, K, N, bits, group_size, int(bool(act_order)), ctypes.byref(plan))
    if rc != OK:
        raise GptqHipError(rc, f"gptq_hip_select(M={M}, K={K}, N={N}, bits={bits}, group_size={group_size})")
    return plan


def build_id() -> str:
    """The digest of the sources the loaded kernel library was built from."""
    return lib().gptq_hip_build_id().decode()


def select_tiled(M: int, K: int, N: int, bits: int, group_size: int, decode: bool = False) -> Plan:
    """The plan of the tiled family; ``decode=True`` asks for its decode kernel (M <= 8) whatever M."""
    plan = Plan()
    fn = lib().gptq_hip_select_tiled_decode if decode else lib().gptq_hip_select_tiled
    rc = fn(M, K, N, bits, group_size, ctypes.byref(plan))
    if rc != OK:
        raise GptqHipError(rc, f"gptq_hip_select_tiled(M={M}, K={K}, N={N}, bits={bits}, group_size={group_size})")
    return plan


def select_route(M: int, K: int, N: int, bits: int, group_size: int, act_order: bool,
                 copies: int = COPY_CHECKPOINT | COPY_SORTED | COPY_TILED, switch_rows=None) -> Route:
    """Which copy of a layer a call with M rows runs on, and the plan there (gptq_hip_select_route).
    ``switch_rows``: (tiled, checkpoint, checkpoint with an activation order) rows from which the library GEMM
    takes over, 0 = never; None = the library's defaults."""
    route = Route()
    sw = None if switch_rows is None else (ctypes.c_int * 3)(*[int(v or 0) for v in switch_rows])
    rc = lib().gptq_hip_select_route(M, K, N, bits, group_size, int(bool(act_order)), copies, sw, ctypes.byref(route))
    if rc != OK:
        raise GptqHipError(rc, f"gptq_hip_select_route(M={M}, K={K}, N={N}, bits={bits}, group_size={group_size}, "
                               f"copies={copies})")
    return route


def select_tiled_transposed(M: int, K: int, N: int, bits: int, group_size: int) -> Plan:
    """The plan of the transposed product gx[M, K] = gy[M, N] @ W^T on the tiled family."""
    plan = Plan()
    rc = lib().gptq_hip_select_tiled_transposed(M, K, N, bits, group_size, ctypes.byref(plan))
    if rc != OK:
        raise GptqHipError(rc, f"gptq_hip_select_tiled_transposed(M={M}, K={K}, N={N}, bits={bits}, "
                               f"group_size={group_size})")
    return plan


def plan_for(kernel: int, M: int, K: int, N: int, bits: int, group_size: int, act_order: bool,
             split_k: int = 0, waves_n: int = 0) -> Plan:
    """Plan of one kernel family with ``split_k`` / ``waves_n`` forced (0 = dispatcher's choice)."""
    plan = Plan()
    rc = lib().gptq_hip_plan_for(kernel, M, K, N, bits, group_size, int(bool(act_order)), split_k, waves_n,
                                 ctypes.byref(plan))
    if rc != OK:
        raise GptqHipError(rc, f"gptq_hip_plan_for(kernel={kernel}, M={M}, K={K}, N={N}, bits={bits}, "
                               f"group_size={group_size}, split_k={split_k}, waves_n={waves_n})")
    return plan
