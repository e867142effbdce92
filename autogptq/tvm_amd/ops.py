"""Torch-tensor front end of the C ABI: pointer plumbing and argument checks only."""
from __future__ import annotations

import ctypes
import os
from typing import Optional

import torch

from . import _lib


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else ctypes.c_void_p(t.data_ptr())


def _need_gpu(name: str, t: torch.Tensor, dtype: torch.dtype):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor")
    if t.device.type != "cuda":
        raise RuntimeError(
            f"{name} is on {t.device}: the GPTQ kernels run on a ROCm GPU only and there is no CPU fallback"
        )
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")


def _stream(device: torch.device):
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


FUSED_BITS = (3, 4)        # widths the matmul kernels on the checkpoint layout (and its sorted copy) cover
FORMAT_BITS = (2, 3, 4, 8)  # widths of the checkpoint format; all four run fused on the tiled format


def check_shapes(qweight, qzeros, scales, g_idx, bias, bits: int, group_size: int, widths=FUSED_BITS):
    if bits not in widths:
        raise NotImplementedError(f"Only {', '.join(map(str, widths))} bits are supported here.")
    rows, N = qweight.shape
    if rows * 32 % bits != 0:
        raise ValueError(f"qweight has {rows} rows, not a multiple of bits={bits} words per 32 channels")
    K = rows * 32 // bits
    gs = K if group_size == -1 else group_size
    if gs <= 0:
        raise ValueError(f"group_size must be -1 or positive, got {group_size}")
    G = (K + gs - 1) // gs
    if K % 32 != 0 or N % 32 != 0:
        raise ValueError(f"infeatures ({K}) and outfeatures ({N}) must be multiples of 32")
    if tuple(scales.shape) != (G, N):
        raise ValueError(f"scales must be [{G}, {N}], got {tuple(scales.shape)}")
    if tuple(qzeros.shape) != (G, N // 32 * bits):
        raise ValueError(f"qzeros must be [{G}, {N // 32 * bits}], got {tuple(qzeros.shape)}")
    if g_idx is not None and tuple(g_idx.shape) != (K,):
        raise ValueError(f"g_idx must be [{K}], got {tuple(g_idx.shape)}")
    if bias is not None and tuple(bias.shape) != (N,):
        raise ValueError(f"bias must be [{N}], got {tuple(bias.shape)}")
    return K, N, G


_workspaces = {}


def _workspace(device: torch.device, nbytes: int, kind: int = 0) -> torch.Tensor:
    """A zero-initialised workspace per (device, stream) and kind, grown on demand.  The kernels leave
    its counters at zero, so it is cleared only when it is (re)allocated.  kind 1: the decode plans of the
    tiled family with halved tiles, whose kernel keeps ALL their bytes zero between launches (the slots through
    which the two halves of a tile meet); they do not share the workspace other plans pack x or partial sums into."""
    key = (device.index, torch.cuda.current_stream(device).cuda_stream, kind)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.zeros(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def gemm(x: torch.Tensor, qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
         g_idx: Optional[torch.Tensor], bias: Optional[torch.Tensor], bits: int, group_size: int,
         plan: Optional[_lib.Plan] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[M, N] fp16 = x[M, K] @ W (+ bias); ``g_idx=None`` means contiguous groups (k // group_size)."""
    _need_gpu("x", x, torch.float16)
    _need_gpu("qweight", qweight, torch.int32)
    _need_gpu("qzeros", qzeros, torch.int32)
    _need_gpu("scales", scales, torch.float16)
    if g_idx is not None:
        _need_gpu("g_idx", g_idx, torch.int32)
    if bias is not None:
        _need_gpu("bias", bias, torch.float16)
    K, N, _ = check_shapes(qweight, qzeros, scales, g_idx, bias, bits, group_size)
    if x.dim() != 2 or x.shape[1] != K:
        raise ValueError(f"x must be [M, {K}], got {tuple(x.shape)}")
    M = x.shape[0]
    dev = x.device
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=dev)
    else:
        _need_gpu("out", out, torch.float16)
        if tuple(out.shape) != (M, N):
            raise ValueError(f"out must be [{M}, {N}]")
    if M == 0:
        return out
    if plan is None:
        plan = _lib.select(M, K, N, bits, group_size, g_idx is not None)
    ws = _workspace(dev, plan.workspace_bytes) if plan.workspace_bytes else None
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_gemm_plan(
            _ptr(x), _ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(g_idx), _ptr(bias), _ptr(out),
            _ptr(ws), ws.numel() if ws is not None else 0, M, K, N, bits, group_size,
            ctypes.byref(plan), _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_gemm(M={M}, K={K}, N={N}, bits={bits}, group_size={group_size})")
    return out


SORTED_MAX_ROWS = 16


def sorted_plan(M: int, K: int, N: int, bits: int, group_size: int) -> Optional[_lib.Plan]:
    """The plan ``gemm_sorted`` would run, or None when the sorted path does not cover the problem (it is for
    decode sizes: the GROUPED family, or up to ``SORTED_MAX_ROWS`` rows on the STREAM kernel that reads x itself):
    the library's rule (gptq_hip_select_route with only the sorted copy on offer)."""
    try:
        r = _lib.select_route(M, K, N, bits, group_size, True, copies=_lib.COPY_SORTED, switch_rows=(0, 0, 0))
    except _lib.GptqHipError:
        return None
    return r.plan if r.copy == _lib.ROUTE_SORTED else None


def gemm_sorted(x: torch.Tensor, qweight_sorted: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
                kmap: torch.Tensor, bias: Optional[torch.Tensor], bits: int, group_size: int,
                plan: Optional[_lib.Plan] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``gemm`` for an activation-order layer whose channels ``pack.sort_channels_by_group`` sorted by
    group; ``x`` and the result are in the layer's original channel order.  M <= ``SORTED_MAX_ROWS``."""
    _need_gpu("x", x, torch.float16)
    _need_gpu("qweight_sorted", qweight_sorted, torch.int32)
    _need_gpu("qzeros", qzeros, torch.int32)
    _need_gpu("scales", scales, torch.float16)
    _need_gpu("kmap", kmap, torch.int32)
    if bias is not None:
        _need_gpu("bias", bias, torch.float16)
    K, N, _ = check_shapes(qweight_sorted, qzeros, scales, None, bias, bits, group_size)
    if tuple(kmap.shape) != (2 * K,):
        raise ValueError(f"kmap must be [{2 * K}], got {tuple(kmap.shape)}")
    if x.dim() != 2 or x.shape[1] != K:
        raise ValueError(f"x must be [M, {K}], got {tuple(x.shape)}")
    M = x.shape[0]
    dev = x.device
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=dev)
    if M == 0:
        return out
    if plan is None:
        plan = sorted_plan(M, K, N, bits, group_size)
        if plan is None:
            raise _lib.GptqHipError(_lib.ERR_UNSUPPORTED, f"gptq_hip_gemm_sorted(M={M}, K={K}, N={N}, bits={bits})")
    ws_bytes = plan.workspace_bytes
    if plan.kernel == _lib.KERNEL_STREAM or (plan.kernel == _lib.KERNEL_GROUPED and M >= 2):
        # kernels that want x in the sorted order (STREAM, GROUPED with packed rows): a small pass puts it
        # behind what the plan itself uses
        ws_bytes = max(ws_bytes, _lib.lib().gptq_hip_sorted_workspace_bytes(M, K, N, bits, group_size))
    ws = _workspace(dev, ws_bytes) if ws_bytes else None
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_gemm_sorted(
            _ptr(x), _ptr(qweight_sorted), _ptr(qzeros), _ptr(scales), _ptr(kmap), _ptr(bias), _ptr(out),
            _ptr(ws), ws.numel() if ws is not None else 0, M, K, N, bits, group_size,
            ctypes.byref(plan), _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_gemm_sorted(M={M}, K={K}, N={N}, bits={bits}, group_size={group_size})")
    return out


def sort_channels(qweight: torch.Tensor, g_idx: torch.Tensor, bits: int, group_size: int):
    """``pack.sort_channels_by_group`` on the library's own kernels: ``(qweight_sorted, kmap)`` on the GPU.
    The caller vouches that every group has exactly ``group_size`` channels."""
    _need_gpu("qweight", qweight, torch.int32)
    _need_gpu("g_idx", g_idx, torch.int32)
    rows, N = qweight.shape
    K = rows * 32 // bits
    if tuple(g_idx.shape) != (K,):
        raise ValueError(f"g_idx must be [{K}], got {tuple(g_idx.shape)}")
    dev = qweight.device
    out = torch.empty_like(qweight)
    kmap = torch.empty(2 * K, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_sort_channels(_ptr(qweight), _ptr(g_idx), _ptr(out), _ptr(kmap), K, N, bits,
                                               group_size, _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_sort_channels(K={K}, N={N}, bits={bits}, group_size={group_size})")
    return out, kmap


def tile_prepare(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor, g_idx: Optional[torch.Tensor],
                 bits: int, group_size: int):
    """``pack.tile_layout`` on the library's own kernels (gptq_hip_tile_prepare): ``(qtile int32 1-D,
    sz int32 [G, N], xsrc int32 [Kp], kinv int16 [K] holding unsigned 16-bit positions)`` on the GPU.  The caller vouches that every group has exactly
    ``group_size`` channels.  Raises ``GptqHipError`` (UNSUPPORTED) for layers the tiled format does not cover."""
    _need_gpu("qweight", qweight, torch.int32)
    _need_gpu("qzeros", qzeros, torch.int32)
    _need_gpu("scales", scales, torch.float16)
    if g_idx is not None:
        _need_gpu("g_idx", g_idx, torch.int32)
    K, N, G = check_shapes(qweight, qzeros, scales, g_idx, None, bits, group_size, widths=FORMAT_BITS)
    dev = qweight.device
    nbytes = _lib.lib().gptq_hip_tiled_bytes(K, N, bits)
    qtile = torch.empty(nbytes // 4, dtype=torch.int32, device=dev)
    sz = torch.empty((G, N), dtype=torch.int32, device=dev)
    xsrc = torch.empty((K + 63) // 64 * 64, dtype=torch.int32, device=dev)
    kinv = torch.empty(K, dtype=torch.int16, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_tile_prepare(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(g_idx), _ptr(qtile),
                                              _ptr(sz), _ptr(xsrc), _ptr(kinv), K, N, bits, group_size, _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_tile_prepare(K={K}, N={N}, bits={bits}, group_size={group_size})")
    return qtile, sz, xsrc, kinv


def gemm_tiled(x: torch.Tensor, qtile: torch.Tensor, sz: torch.Tensor, xsrc: Optional[torch.Tensor],
               kinv: Optional[torch.Tensor], bias: Optional[torch.Tensor], bits: int, group_size: int,
               plan: Optional[_lib.Plan] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[M, N] fp16 = x[M, K] @ W (+ bias) on a layer in the tiled format (``tile_prepare``); x and y in the
    layer's own channel order; ``xsrc = kinv = None`` means no activation order."""
    _need_gpu("x", x, torch.float16)
    _need_gpu("qtile", qtile, torch.int32)
    _need_gpu("sz", sz, torch.int32)
    if (xsrc is None) != (kinv is None):
        raise ValueError("xsrc and kinv go together: pass both (activation order) or neither")
    if xsrc is not None:
        _need_gpu("xsrc", xsrc, torch.int32)
        _need_gpu("kinv", kinv, torch.int16)
    if bias is not None:
        _need_gpu("bias", bias, torch.float16)
    if x.dim() != 2 or sz.dim() != 2:
        raise ValueError("x must be [M, K] and sz [G, N]")
    M, K = x.shape
    G, N = sz.shape
    Kp = (K + 63) // 64 * 64
    if qtile.numel() * 4 != Kp * N * bits // 8:
        raise ValueError(f"qtile holds {qtile.numel() * 4} bytes, a {K} x {N} layer of {bits} bits needs {Kp * N * bits // 8}")
    if xsrc is not None and (tuple(xsrc.shape) != (Kp,) or tuple(kinv.shape) != (K,)):
        raise ValueError(f"xsrc must be [{Kp}] and kinv [{K}], got {tuple(xsrc.shape)} and {tuple(kinv.shape)}")
    if bias is not None and tuple(bias.shape) != (N,):
        raise ValueError(f"bias must be [{N}], got {tuple(bias.shape)}")
    dev = x.device
    if out is None:
        out = torch.empty((M, N), dtype=torch.float16, device=dev)
    if M == 0:
        return out
    if plan is None:
        plan = _lib.select_tiled(M, K, N, bits, group_size)
    slots = bool(plan.flags & _lib.PLAN_PRIVATE_ZERO_WORKSPACE)   # (halved tiles: a workspace of their own)
    ws = _workspace(dev, plan.workspace_bytes, 1 if slots else 0) if plan.workspace_bytes else None
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_gemm_tiled(_ptr(x), _ptr(qtile), _ptr(sz), _ptr(xsrc), _ptr(kinv), _ptr(bias), _ptr(out),
                                            _ptr(ws), ws.numel() if ws is not None else 0, M, K, N, bits, group_size,
                                            ctypes.byref(plan), _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_gemm_tiled(M={M}, K={K}, N={N}, bits={bits}, group_size={group_size})")
    return out


def tile_prepare_transposed(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
                            xsrc: Optional[torch.Tensor], bits: int, group_size: int):
    """``pack.tile_layout_transposed`` on the library's own kernels (gptq_hip_tile_prepare_transposed): the copy the
    transposed product runs on, ``(qtile_t int32 1-D, szt int32 [G, ceil64(N) / 8, 8])``.  ``xsrc``: the map
    ``tile_prepare`` returned for the layer (the channel at each sorted position), None without an activation
    order."""
    _need_gpu("qweight", qweight, torch.int32)
    _need_gpu("qzeros", qzeros, torch.int32)
    _need_gpu("scales", scales, torch.float16)
    K, N, G = check_shapes(qweight, qzeros, scales, None, None, bits, group_size, widths=FORMAT_BITS)
    if xsrc is not None:
        _need_gpu("xsrc", xsrc, torch.int32)
        if tuple(xsrc.shape) != ((K + 63) // 64 * 64,):
            raise ValueError(f"xsrc must be [{(K + 63) // 64 * 64}], got {tuple(xsrc.shape)}")
    dev = qweight.device
    lib = _lib.lib()
    qtile_t = torch.empty(lib.gptq_hip_tiled_transposed_bytes(K, N, bits) // 4, dtype=torch.int32, device=dev)
    szt = torch.empty((G, (N + 63) // 64 * 8, 8), dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        rc = lib.gptq_hip_tile_prepare_transposed(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(xsrc), _ptr(qtile_t),
                                                  _ptr(szt), K, N, bits, group_size, _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_tile_prepare_transposed(K={K}, N={N}, bits={bits}, "
                                    f"group_size={group_size})")
    return qtile_t, szt


def gemm_tiled_transposed(gy: torch.Tensor, qtile_t: torch.Tensor, szt: torch.Tensor, xsrc: Optional[torch.Tensor],
                          K: int, bits: int, group_size: int, plan: Optional[_lib.Plan] = None,
                          out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """gx[M, K] fp16 = gy[M, N] @ W^T on the transposed tiled copy (``tile_prepare_transposed``): the gradient of
    ``y = x @ W`` with respect to x (the reference's transpose_matmul248, qlinear_triton.py:298-317); gy and gx in
    the layer's own channel order."""
    _need_gpu("gy", gy, torch.float16)
    _need_gpu("qtile_t", qtile_t, torch.int32)
    _need_gpu("szt", szt, torch.int32)
    if xsrc is not None:
        _need_gpu("xsrc", xsrc, torch.int32)
    if gy.dim() != 2 or szt.dim() != 3:
        raise ValueError("gy must be [M, N] and szt [G, ceil64(N) / 8, 8]")
    M, N = gy.shape
    Np = (N + 63) // 64 * 64
    gs = K if group_size == -1 else group_size
    if K % 32 != 0 or N % 32 != 0 or K % gs != 0:
        raise ValueError(f"a {K} x {N} layer with groups of {gs} is not one the tiled format covers")
    if qtile_t.numel() * 4 != K * Np * bits // 8:
        raise ValueError(f"qtile_t holds {qtile_t.numel() * 4} bytes, a {K} x {N} layer of {bits} bits needs "
                         f"{K * Np * bits // 8}")
    if tuple(szt.shape) != (K // gs, Np // 8, 8):
        raise ValueError(f"szt must be [{K // gs}, {Np // 8}, 8], got {tuple(szt.shape)}")
    if xsrc is not None and tuple(xsrc.shape) != ((K + 63) // 64 * 64,):
        raise ValueError(f"xsrc must be [{(K + 63) // 64 * 64}], got {tuple(xsrc.shape)}")
    dev = gy.device
    if out is None:
        out = torch.empty((M, K), dtype=torch.float16, device=dev)
    if M == 0:
        return out
    if plan is None:
        plan = _lib.select_tiled_transposed(M, K, N, bits, group_size)
    ws = _workspace(dev, plan.workspace_bytes)
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_gemm_tiled_transposed(_ptr(gy), _ptr(qtile_t), _ptr(szt), _ptr(xsrc), _ptr(out), _ptr(ws),
                                                       ws.numel(), M, K, N, bits, group_size, ctypes.byref(plan),
                                                       _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_gemm_tiled_transposed(M={M}, K={K}, N={N}, bits={bits}, "
                                    f"group_size={group_size})")
    return out


def tiled_wins(M: int, K: int, N: int, act_order: bool, bits: int = 4, one_group: bool = False) -> bool:
    """Whether a call with M rows runs on the tiled copy of a layer that holds all three copies (group size 128,
    or one group): the library's own rule (gptq_hip_select_route), where the measurements behind it are kept."""
    gs = -1 if one_group else 128
    return _lib.select_route(M, K, N, bits, gs, act_order, switch_rows=(0, 0, 0)).copy == _lib.ROUTE_TILED


def dequant(qweight: torch.Tensor, qzeros: torch.Tensor, scales: torch.Tensor,
            g_idx: Optional[torch.Tensor], bits: int, group_size: int) -> torch.Tensor:
    """The materialised fp16 weight [K, N], bit-exact with the reference's dequantisation."""
    _need_gpu("qweight", qweight, torch.int32)
    _need_gpu("qzeros", qzeros, torch.int32)
    _need_gpu("scales", scales, torch.float16)
    if g_idx is not None:
        _need_gpu("g_idx", g_idx, torch.int32)
    K, N, _ = check_shapes(qweight, qzeros, scales, g_idx, None, bits, group_size, widths=FORMAT_BITS)
    dev = qweight.device
    w = torch.empty((K, N), dtype=torch.float16, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.lib().gptq_hip_dequant(_ptr(qweight), _ptr(qzeros), _ptr(scales), _ptr(g_idx), _ptr(w),
                                         K, N, bits, group_size, _stream(dev))
    if rc != _lib.OK:
        raise _lib.GptqHipError(rc, f"gptq_hip_dequant(K={K}, N={N}, bits={bits})")
    return w


# ---------------------------------------------------------------------------------------------
# torch.ops.gptq_hip.{gemm, gemm_sorted, gemm_tiled, dequant}: the same calls as dispatcher-visible
# operators.  csrc/binding.cpp defines them in C++ (libgptq_hip_torch.so, built beside the kernel library);
# only GPU kernels and shape-only "meta" versions exist; a CPU tensor raises ("no CPU fallback").  Without the built operator library the same operators are registered from here, as thin
# wrappers of the functions above (ctypes into the same C ABI).
def _meta_gemm(x, qweight, qzeros, scales, g_idx, bias, bits, group_size):
    return x.new_empty((x.shape[0], qweight.shape[1]), dtype=torch.float16)


def _meta_gemm_sorted(x, qweight_sorted, qzeros, scales, kmap, bias, bits, group_size):
    return x.new_empty((x.shape[0], qweight_sorted.shape[1]), dtype=torch.float16)


def _meta_gemm_tiled(x, qtile, sz, xsrc, kinv, bias, bits, group_size):
    return x.new_empty((x.shape[0], sz.shape[1]), dtype=torch.float16)


def _meta_dequant(qweight, qzeros, scales, g_idx, bits, group_size):
    return scales.new_empty((qweight.shape[0] * 32 // bits, qweight.shape[1]), dtype=torch.float16)


BINDING_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "csrc", "libgptq_hip_torch.so")
NATIVE_OPS = False   # True when torch.ops.gptq_hip.* are the C++ operators


def _register_torch_ops():
    global NATIVE_OPS
    keep = []
    native = False
    if os.path.exists(BINDING_PATH) and os.path.exists(_lib.LIB_PATH):
        try:
            _lib.lib()                  # the kernel library first (checks that it matches its sources)
            native = True
        except RuntimeError:
            pass                        # stale: the Python operators below report it on their first call
    if native:
        torch.ops.load_library(BINDING_PATH)
        built = torch.ops.gptq_hip.binding_build_id()
        if built != _lib.build_id():
            raise RuntimeError(f"{BINDING_PATH} was built from other sources ({built}) than the kernel library "
                               f"({_lib.build_id()}): run python -m autogptq.tvm_amd.build")
        NATIVE_OPS = True
    else:
        lib = torch.library.Library("gptq_hip", "DEF")
        lib.define("gemm(Tensor x, Tensor qweight, Tensor qzeros, Tensor scales, Tensor? g_idx, Tensor? bias, "
                   "int bits, int group_size) -> Tensor")
        lib.define("gemm_sorted(Tensor x, Tensor qweight_sorted, Tensor qzeros, Tensor scales, Tensor kmap, "
                   "Tensor? bias, int bits, int group_size) -> Tensor")
        lib.define("gemm_tiled(Tensor x, Tensor qtile, Tensor sz, Tensor? xsrc, Tensor? kinv, Tensor? bias, "
                   "int bits, int group_size) -> Tensor")
        lib.define("dequant(Tensor qweight, Tensor qzeros, Tensor scales, Tensor? g_idx, int bits, int group_size) "
                   "-> Tensor")
        lib.impl("gemm", lambda x, qw, qz, sc, g, b, bits, gs: gemm(x, qw, qz, sc, g, b, bits, gs), "CUDA")
        lib.impl("gemm_sorted", lambda x, qw, qz, sc, km, b, bits, gs: gemm_sorted(x, qw, qz, sc, km, b, bits, gs), "CUDA")
        lib.impl("gemm_tiled", lambda x, qt, sz, xs, ki, b, bits, gs: gemm_tiled(x, qt, sz, xs, ki, b, bits, gs), "CUDA")
        lib.impl("dequant", lambda qw, qz, sc, g, bits, gs: dequant(qw, qz, sc, g, bits, gs), "CUDA")
        # CPU tensors reach the same functions, whose first check raises ("no CPU fallback")
        lib.impl("gemm", lambda x, qw, qz, sc, g, b, bits, gs: gemm(x, qw, qz, sc, g, b, bits, gs), "CPU")
        lib.impl("gemm_sorted", lambda x, qw, qz, sc, km, b, bits, gs: gemm_sorted(x, qw, qz, sc, km, b, bits, gs), "CPU")
        lib.impl("gemm_tiled", lambda x, qt, sz, xs, ki, b, bits, gs: gemm_tiled(x, qt, sz, xs, ki, b, bits, gs), "CPU")
        lib.impl("dequant", lambda qw, qz, sc, g, bits, gs: dequant(qw, qz, sc, g, bits, gs), "CPU")
        keep.append(lib)
    meta = torch.library.Library("gptq_hip", "IMPL", "Meta")
    meta.impl("gemm", _meta_gemm)
    meta.impl("gemm_sorted", _meta_gemm_sorted)
    meta.impl("gemm_tiled", _meta_gemm_tiled)
    meta.impl("dequant", _meta_dequant)
    keep.append(meta)
    return keep


_TORCH_OPS = _register_torch_ops()  # kept alive for the life of the module
