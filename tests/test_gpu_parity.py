"""GPU parity tests: the HIP kernels, called through the C ABI (ctypes -> libgptq_hip.so),
against the CPU oracle on the same seeded inputs.

Bars: dequantised weights bit-exact; outputs within rtol = atol = 1e-2 of x @ W (W the oracle's
fp16 weight, fp32-or-wider accumulation).  Tighter internal bounds are also asserted so that an
indexing slip cannot hide inside the contract's tolerance.
"""
import ctypes

import numpy as np
import pytest
import torch

from autogptq.tvm_amd import QuantLinear, _lib, ops, pack
from tests.parity_util import (ATOL, RTOL, assert_close, assert_tight, expected_output, expected_weight, layer,
                               to_dev)

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def run_gemm(D, g_idx="auto", plan=None, x=None):
    g = D["g_idx"] if (g_idx == "auto" and D["desc_act"]) else (None if g_idx == "auto" else g_idx)
    return ops.gemm(D["x"] if x is None else x, D["qweight"], D["qzeros"], D["scales"], g, D.get("bias"),
                    D["bits"], D["group_size"], plan=plan)


# ------------------------------------------------------------------ dequant: bit-exact
@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("shape", [(64, 32, 32), (256, 96, 64), (4096, 256, 128), (1024, 160, -1)])
def test_dequant_bit_exact_small(dev, bits, desc_act, shape):
    K, N, gs = shape
    L = layer(100 + bits, K, N, bits, gs, desc_act)
    D = to_dev(L, dev)
    for g in (D["g_idx"], None if not desc_act else D["g_idx"]):
        w = ops.dequant(D["qweight"], D["qzeros"], D["scales"], g, bits, gs).cpu()
        want = expected_weight(L)
        assert torch.equal(w.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("bits,K,N,gs,desc_act", [
    (4, 4096, 4096, 128, False),      # config 1
    (3, 4096, 11008, 128, True),      # config 2
    (4, 11008, 4096, 128, True),      # config 3/4 down projection
    (3, 9216, 9216, -1, True),        # config 5 attention
])
def test_dequant_bit_exact_full_size(dev, bits, K, N, gs, desc_act):
    L = layer(200 + bits, K, N, bits, gs, desc_act)
    D = to_dev(L, dev)
    w = ops.dequant(D["qweight"], D["qzeros"], D["scales"], D["g_idx"], bits, gs).cpu()
    want = expected_weight(L)
    assert torch.equal(w.view(torch.int16), want.view(torch.int16))


def test_dequant_extreme_scales_bit_exact(dev):
    # subnormal, tiny, large and negative fp16 scales: the single rounding must still match
    L = layer(7, 128, 64, 4, 32, True)
    pats = torch.tensor([0x0001, 0x03FF, 0x0400, 0x1234, 0x7BFF, 0x8001, 0xB555, 0xFBFF, 0x0000, 0x3C00],
                        dtype=torch.int32).to(torch.int16)
    flat = L["scales"].view(torch.int16).flatten()
    flat[: 10 * (flat.numel() // 10)] = pats.repeat(flat.numel() // 10)
    D = to_dev(L, dev)
    w = ops.dequant(D["qweight"], D["qzeros"], D["scales"], D["g_idx"], 4, 32).cpu()
    assert torch.equal(w.view(torch.int16), expected_weight(L).view(torch.int16))


# ------------------------------------------------------------------ matmul: small shapes, all the edges
M_EDGES = [1, 2, 3, 5, 8, 15, 16, 17, 31, 33, 64, 65, 127, 129, 257]


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("M", M_EDGES)
def test_gemm_ragged_m(dev, bits, desc_act, M):
    L = layer(300 + M, 512, 192, bits, 128, desc_act, M=M, bias=(M % 2 == 1))
    D = to_dev(L, dev)
    y = run_gemm(D)
    assert y.shape == (M, 192) and y.dtype == torch.float16
    assert_close(y, expected_output(L), f"bits={bits} act={desc_act} M={M}")
    assert_tight(y, expected_output(L), f"bits={bits} act={desc_act} M={M}")


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(32, 32, 32), (96, 32, 32), (160, 96, -1), (384, 64, 64), (1024, 416, 32),
                                    (2048, 1056, 256)])
@pytest.mark.parametrize("M", [1, 7, 40])
def test_gemm_odd_shapes(dev, bits, K, N, gs, M):
    for desc_act in (False, True):
        L = layer(400 + K + N, K, N, bits, gs, desc_act, M=M)
        D = to_dev(L, dev)
        y = run_gemm(D)
        assert_close(y, expected_output(L), f"bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
        assert_tight(y, expected_output(L), f"bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")


@pytest.mark.parametrize("bits", [3, 4])
def test_gemm_explicit_contiguous_g_idx_equals_null(dev, bits):
    L = layer(55, 512, 128, bits, 64, False, M=4)
    D = to_dev(L, dev)
    a = run_gemm(D, g_idx=None)
    b = run_gemm(D, g_idx=D["g_idx"])
    assert_close(a, expected_output(L), "null g_idx")
    assert_close(b, expected_output(L), "explicit g_idx")


@pytest.mark.parametrize("bits", [3, 4])
def test_gemm_integer_exact(dev, bits):
    # x = 1, scales = 1, one group: y[n] = sum_k (q - z), exactly representable -> must be exact
    L = layer(66, 64, 64, bits, -1, False, M=2)  # |sum| <= 64 * 16 < 2048: exact in fp16
    L["scales"] = torch.ones_like(L["scales"])
    L["x"] = torch.ones_like(L["x"])
    D = to_dev(L, dev)
    y = run_gemm(D).float().cpu()
    want = (L["codes"].numpy() - L["zeros"].numpy()[0][None, :]).sum(axis=0).astype(np.float32)
    assert np.array_equal(y[0].numpy(), want) and np.array_equal(y[1].numpy(), want)


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("waves,split", [(1, 1), (2, 1), (4, 1), (8, 1), (1, 3), (4, 2), (8, 2)])
@pytest.mark.parametrize("M", [3, 20, 40, 130])
def test_stream_forced_waves_and_split_k(dev, bits, desc_act, waves, split, M):
    # K = 4096 gives every (waves, split) at least one whole ring of steps per wave; N = 352 ends
    # in a partly filled column tile; M covers every tile height and ragged last M blocks
    K, N = 4096, 352
    L = layer(700 + waves * 10 + split, K, N, bits, 128, desc_act, M=M, bias=True)
    D = to_dev(L, dev)
    plan = _lib.plan_for(_lib.KERNEL_STREAM, M, K, N, bits, 128, desc_act, split_k=split, waves_n=waves)
    assert plan.kernel == _lib.KERNEL_STREAM and plan.waves_k == waves and plan.split_k == split
    y1 = run_gemm(D, plan=plan)
    y2 = run_gemm(D, plan=plan)  # same workspace again: counters left at zero, packed x rewritten
    assert_close(y1, expected_output(L), f"waves={waves} split={split}")
    assert_tight(y1, expected_output(L), f"waves={waves} split={split}")
    assert torch.equal(y1, y2), "result changed between two identical calls"


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(32, 32, 32), (160, 96, -1), (1024, 416, 32), (2048, 1056, 256), (4096, 64, 64)])
@pytest.mark.parametrize("M", [5, 33])
def test_stream_matches_the_tiled_matmul(dev, bits, K, N, gs, M):
    # two independent kernels on two layouts, same exact fp16 weights: they may differ only in summation order
    for desc_act in (False, True):
        L = layer(800 + M, K, N, bits, gs, desc_act, M=M)
        D = to_dev(L, dev)
        a = run_gemm(D, plan=_lib.plan_for(_lib.KERNEL_STREAM, M, K, N, bits, gs, desc_act))
        qtile, sz, xsrc, kinv = ops.tile_prepare(D["qweight"], D["qzeros"], D["scales"],
                                                 D["g_idx"] if desc_act else None, bits, gs)
        b = ops.gemm_tiled(D["x"], qtile, sz, xsrc if desc_act else None, kinv if desc_act else None, None, bits, gs)
        assert_close(a, expected_output(L), "stream")
        assert_close(b, expected_output(L), "tiled")
        assert_tight(a, b.float().cpu(), "stream vs tiled")


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("split", [1, 2, 5, 16])
def test_grouped_forced_split_k(dev, bits, desc_act, M, split):
    K, N, gs = 2048, 320, 128
    L = layer(600 + split, K, N, bits, gs, desc_act, M=M, bias=True)
    D = to_dev(L, dev)
    try:
        plan = _lib.plan_for(_lib.KERNEL_GROUPED, M, K, N, bits, gs, desc_act, split_k=split)
    except _lib.GptqHipError as e:
        assert e.status == _lib.ERR_UNSUPPORTED  # e.g. the LDS operand of an unsplit K range
        pytest.skip("this split is outside the GROUPED family for the shape")
    assert plan.kernel == _lib.KERNEL_GROUPED
    y1 = run_gemm(D, plan=plan)
    y2 = run_gemm(D, plan=plan)
    assert_close(y1, expected_output(L), f"grouped split={split}")
    assert_tight(y1, expected_output(L), f"grouped split={split}")
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(512, 96, 128), (1024, 416, 32), (2048, 1056, 256), (4096, 352, 128), (1024, 160, -1),
                                    (11008, 256, 128), (4096, 16480, 128)])
@pytest.mark.parametrize("M", [2, 3, 4, 5, 7, 8])
def test_grouped_packed_rows(dev, bits, K, N, gs, M):
    """Two to four rows in one operand tile of the GROUPED kernel, five to eight in two (contiguous groups):
    against the oracle, against the STREAM kernel on the same inputs, and with a forced split of K."""
    L = layer(760 + K + M, K, N, bits, gs, False, M=M, bias=True)
    D = to_dev(L, dev)
    if M == 2:
        # (a forced GROUPED plan for two rows is the unpacked one; the dispatcher prefers the packed one)
        plan = _lib.select(M, K, N, bits, gs, False)
        if not (plan.kernel == _lib.KERNEL_GROUPED and plan.row_tiles == 4):
            pytest.skip("no packed-row plan for the shape")
    else:
        try:
            plan = _lib.plan_for(_lib.KERNEL_GROUPED, M, K, N, bits, gs, False)
        except _lib.GptqHipError as e:
            assert e.status == _lib.ERR_UNSUPPORTED   # e.g. more than four groups in a wave's K range
            pytest.skip("no packed-row plan for the shape")
    assert plan.kernel == _lib.KERNEL_GROUPED and plan.row_tiles == (4 if M <= 4 else 8)
    want = expected_output(L)
    y = run_gemm(D, plan=plan)
    assert_close(y, want, "packed rows")
    assert_tight(y, want, "packed rows")
    assert torch.equal(y, run_gemm(D, plan=plan))
    assert_tight(y, run_gemm(D, plan=_lib.plan_for(_lib.KERNEL_STREAM, M, K, N, bits, gs, False)).cpu(), "packed rows vs STREAM")
    assert_close(run_gemm(D), want, "dispatcher's choice")
    for split in (2, 4):
        try:
            ps = _lib.plan_for(_lib.KERNEL_GROUPED, M, K, N, bits, gs, False, split_k=split)
        except _lib.GptqHipError:
            continue
        ys = run_gemm(D, plan=ps)
        assert_close(ys, want, f"packed rows split={split}")
        assert_tight(ys, want, f"packed rows split={split}")


def test_grouped_packed_rows_rejects_what_it_cannot_hold(dev):
    # an activation order, or a ninth row, is outside the packed-row plans
    with pytest.raises(_lib.GptqHipError) as e:
        _lib.plan_for(_lib.KERNEL_GROUPED, 4, 1024, 128, 4, 128, True)
    assert e.value.status == _lib.ERR_UNSUPPORTED
    with pytest.raises(_lib.GptqHipError) as e:
        _lib.plan_for(_lib.KERNEL_GROUPED, 9, 1024, 128, 4, 128, False)
    assert e.value.status == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("N,wn", [(16480, 2), (32864, 4)])
def test_grouped_wide_workgroups(dev, bits, desc_act, M, N, wn):
    # 257..512 column tiles: the dispatcher gives a workgroup 128 columns (two waves along N); more: 256
    K, gs = 512, 128
    L = layer(650 + bits + M, K, N, bits, gs, desc_act, M=M, bias=True)
    D = to_dev(L, dev)
    plan = _lib.select(M, K, N, bits, gs, desc_act)
    if plan.kernel == _lib.KERNEL_GROUPED:
        assert plan.waves_n == wn and plan.grid_x == (N + 64 * wn - 1) // (64 * wn)
    y = run_gemm(D)
    assert_close(y, expected_output(L), "wide workgroups")
    assert_tight(y, expected_output(L), "wide workgroups")
    if desc_act and ops.sorted_plan(M, K, N, bits, gs) is not None:
        ys = run_sorted(D)
        assert_close(ys, expected_output(L), "wide workgroups, sorted")
        assert_tight(ys, expected_output(L), "wide workgroups, sorted")


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(96, 32, 32), (1024, 416, 32), (2048, 1056, 256), (11008, 256, 128), (4096, 64, 64)])
@pytest.mark.parametrize("M", [1, 2])
def test_grouped_matches_stream(dev, bits, K, N, gs, M):
    """The two kernel families on the same inputs: STREAM forms the reference's rounded fp16
    weights, GROUPED applies scales per group; they must agree far inside the tolerance."""
    for desc_act in (False, True):
        L = layer(700 + K, K, N, bits, gs, desc_act, M=M)
        D = to_dev(L, dev)
        try:
            pg = _lib.plan_for(_lib.KERNEL_GROUPED, M, K, N, bits, gs, desc_act)
        except _lib.GptqHipError:
            continue
        a = run_gemm(D, plan=pg)
        b = run_gemm(D, plan=_lib.plan_for(_lib.KERNEL_STREAM, M, K, N, bits, gs, desc_act))
        want = expected_output(L)
        assert_close(a, want, "grouped")
        assert_close(b, want, "stream")
        assert_tight(a, want, "grouped")
        assert_tight(b, want, "stream")


def test_gemm_does_not_write_outside_y(dev):
    M, K, N = 5, 512, 96
    L = layer(77, K, N, 4, 128, True, M=M)
    D = to_dev(L, dev)
    guard = 4096
    buf = torch.full((guard + M * N + guard,), 1234.0, dtype=torch.float16, device=dev)
    out = buf[guard: guard + M * N].view(M, N)
    ops.gemm(D["x"], D["qweight"], D["qzeros"], D["scales"], D["g_idx"], None, 4, 128, out=out)
    assert_close(out, expected_output(L), "guarded out")
    assert bool((buf[:guard] == 1234.0).all()) and bool((buf[guard + M * N:] == 1234.0).all())


# ------------------------------------------------------------------ the benchmark configurations
FULL = [
    # (name, bits, K, N, gs, desc_act, Ms): every shape x M of the benchmark configurations
    ("c1-int4-4096x4096", 4, 4096, 4096, 128, False, [1, 2, 4, 8]),
    ("c2-int3-4096x11008-act", 3, 4096, 11008, 128, True, [1]),
    ("c3-int4-4096x11008", 4, 4096, 11008, 128, False, [1, 2, 4, 8]),
    ("c3-int4-11008x4096", 4, 11008, 4096, 128, False, [1, 2, 4, 8]),
    ("c4-int4-4096x11008-act", 4, 4096, 11008, 128, True, [16, 64, 128, 256]),
    ("c4-int3-4096x11008-act", 3, 4096, 11008, 128, True, [16, 64, 128, 256]),
    ("c4-int4-11008x4096-act", 4, 11008, 4096, 128, True, [16, 64, 128, 256]),
    ("c4-int3-11008x4096-act", 3, 11008, 4096, 128, True, [16, 64, 128, 256]),
    ("c5-int3-9216x9216-act-g1", 3, 9216, 9216, -1, True, [1, 32]),
    ("c5-int3-9216x36864-act-g1", 3, 9216, 36864, -1, True, [1, 32]),
    ("c5-int3-36864x9216-act-g1", 3, 36864, 9216, -1, True, [1, 32]),
]


@pytest.mark.parametrize("name,bits,K,N,gs,desc_act,Ms", FULL, ids=[f[0] for f in FULL])
def test_gemm_full_size(dev, name, bits, K, N, gs, desc_act, Ms):
    L = layer(7000 + [f[0] for f in FULL].index(name), K, N, bits, gs, desc_act, M=max(Ms))
    D = to_dev(L, dev)
    w16 = expected_weight(L)
    for M in Ms:
        x = L["x"][:M].contiguous()
        y = run_gemm(D, x=x.to(dev))
        want = expected_output(L, x=x, w16=w16)
        assert_close(y, want, f"{name} M={M}")
        assert_tight(y, want, f"{name} M={M}")
        y2 = run_gemm(D, x=x.to(dev))
        assert torch.equal(y, y2), f"{name} M={M}: two identical calls differ"


def test_gemm_linearity_at_full_size(dev):
    # size-independent property: f(a + b) = f(a) + f(b) up to rounding, f(2x) = 2 f(x) exactly
    L = layer(900, 4096, 11008, 3, 128, True, M=2)
    # keep fp16 subnormals out of x: doubling must stay exact on every path, matrix cores included
    L["x"] = torch.where(L["x"].abs() < 1e-3, torch.zeros_like(L["x"]), L["x"])
    D = to_dev(L, dev)
    x = D["x"]
    y = run_gemm(D)
    y2 = run_gemm(D, x=(x * 2).contiguous())
    normal = y.float().abs() >= 2.0 ** -13  # an fp16-subnormal output rounds on a fixed grid, not a relative one
    assert torch.equal(y2.float()[normal], (y.float() * 2)[normal])  # scaling by 2 is exact in fp16 and fp32
    ysum = run_gemm(D, x=(x[0:1] + x[1:2]).contiguous())
    assert_close(ysum, (y[0:1].float() + y[1:2].float()), "additivity", rtol=2e-2, atol=2e-2)


# ------------------------------------------------------------------ the module
# ------------------------------------------------------------------ the other widths of the format: 2 and 8 bits
@pytest.mark.parametrize("bits", [2, 8])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("shape", [(64, 32, 32), (256, 96, 64), (4096, 256, 128), (1024, 160, -1)])
def test_dequant_bit_exact_two_and_eight_bits(dev, bits, desc_act, shape):
    K, N, gs = shape
    L = layer(120 + bits, K, N, bits, gs, desc_act)
    D = to_dev(L, dev)
    w = ops.dequant(D["qweight"], D["qzeros"], D["scales"], D["g_idx"] if desc_act else None, bits, gs).cpu()
    assert torch.equal(w.view(torch.int16), expected_weight(L).view(torch.int16))


@pytest.mark.parametrize("bits", [2, 8])
@pytest.mark.parametrize("M", [1, 7])
def test_module_runs_two_and_eight_bit_layers_as_dequant_plus_gemm(dev, bits, M):
    K, N, gs = 512, 256, 128
    L = layer(130 + bits, K, N, bits, gs, True, M=M, bias=True)
    q = QuantLinear(bits, gs, K, N, True, tile_for_prefill=False)   # (with the tiled copy these widths run fused)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q = q.to(dev)
    assert q.route(M) == "library"
    y = q(L["x"].to(dev))
    assert y.shape == (M, N) and y.dtype == torch.float16
    assert_close(y, expected_output(L), f"module forward, {bits} bits")
    assert torch.equal(q.dequantize().cpu().view(torch.int16), expected_weight(L).view(torch.int16))
    # the entry points on the checkpoint layout do not take these widths
    with pytest.raises(NotImplementedError):
        run_gemm(to_dev(L, dev))


@pytest.mark.parametrize("bits", [3, 4, 8])
@pytest.mark.parametrize("M", [1, 9])
def test_module_gives_a_gradient_for_its_input(dev, bits, M):
    # grad_x = grad_y @ W^T (qlinear_triton.py:195-273), against the oracle's dequantised weight
    K, N, gs = 512, 256, 128
    L = layer(140 + bits, K, N, bits, gs, True, M=M, bias=True)
    q = QuantLinear(bits, gs, K, N, True)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q = q.to(dev)
    x = L["x"].to(dev).requires_grad_(True)
    y = q(x)
    assert y.requires_grad
    assert_close(y, expected_output(L), "forward under autograd")
    gy = torch.randn(M, N, generator=torch.Generator().manual_seed(9)).half()
    y.backward(gy.to(dev))
    want = gy.float() @ expected_weight(L).float().t()
    assert x.grad is not None and x.grad.shape == (M, K)
    assert_close(x.grad, want, "input gradient", rtol=1e-2, atol=2e-2)
    with torch.no_grad():
        assert not q(x).requires_grad


# ------------------------------------------------------------------ activation order, channels sorted at load time
def run_sorted(D, plan=None):
    qs, kmap = pack.sort_channels_by_group(D["qweight"], D["g_idx"], D["bits"], D["group_size"])
    return ops.gemm_sorted(D["x"], qs, D["qzeros"], D["scales"], kmap, D.get("bias"), D["bits"], D["group_size"],
                           plan=plan)


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(96, 32, 32), (1024, 416, 32), (2048, 1056, 256), (11008, 256, 128),
                                    (4096, 64, 64), (4096, 352, 128), (1024, 160, -1)])
@pytest.mark.parametrize("M", [1, 2])
def test_sorted_decode_matches_oracle_and_unsorted_kernel(dev, bits, K, N, gs, M):
    L = layer(900 + K + M, K, N, bits, gs, True, M=M, bias=True)
    D = to_dev(L, dev)
    plan = ops.sorted_plan(M, K, N, bits, gs)
    if plan is None:
        pytest.skip("not a GROUPED problem")
    want = expected_output(L)
    y = run_sorted(D)
    assert_close(y, want, "sorted decode")
    assert_tight(y, want, "sorted decode")
    assert torch.equal(y, run_sorted(D))
    assert_tight(y, run_gemm(D).cpu(), "sorted vs unsorted kernel")


@pytest.mark.parametrize("K,N", [(4096, 11008), (11008, 4096)])
def test_sorted_path_at_full_size(dev, K, N):
    """The benchmark's own path at its own size: gptq_hip_gemm_sorted on the 3-bit activation-order layer,
    decode and small batches, against the oracle and against the unsorted kernels; two calls must agree."""
    bits, gs = 3, 128
    L = layer(7100 + K // 1000, K, N, bits, gs, True, M=16)
    D = to_dev(L, dev)
    w16 = expected_weight(L)
    qs, kmap = ops.sort_channels(D["qweight"], D["g_idx"], bits, gs)
    for M in (1, 2, 8, 16):
        x = L["x"][:M].contiguous()
        xd = x.to(dev)
        assert ops.sorted_plan(M, K, N, bits, gs) is not None
        y = ops.gemm_sorted(xd, qs, D["qzeros"], D["scales"], kmap, None, bits, gs)
        want = expected_output(L, x=x, w16=w16)
        assert_close(y, want, f"sorted {K}x{N} M={M}")
        assert_tight(y, want, f"sorted {K}x{N} M={M}")
        assert torch.equal(y, ops.gemm_sorted(xd, qs, D["qzeros"], D["scales"], kmap, None, bits, gs))
        assert_tight(y, run_gemm(D, x=xd).cpu(), f"sorted vs unsorted {K}x{N} M={M}")


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(1024, 416, 32), (2048, 1056, 256), (11008, 256, 128), (4096, 352, 128), (1024, 160, -1)])
@pytest.mark.parametrize("M", [3, 8, 16])
def test_sorted_small_batch_matches_oracle(dev, bits, K, N, gs, M):
    # up to 16 rows: x is put into the sorted order by a small pass, then the kernel for contiguous groups runs
    L = layer(930 + K + M, K, N, bits, gs, True, M=M, bias=True)
    D = to_dev(L, dev)
    plan = ops.sorted_plan(M, K, N, bits, gs)
    if plan is None:
        pytest.skip("not covered by the sorted path")
    # (three rows may also go to the GROUPED kernel with packed rows, behind the same reordering pass)
    assert (plan.kernel == _lib.KERNEL_STREAM and plan.row_tiles == 1) or \
        (plan.kernel == _lib.KERNEL_GROUPED and M <= 8 and plan.row_tiles == (4 if M <= 4 else 8))
    want = expected_output(L)
    y = run_sorted(D)
    assert_close(y, want, "sorted small batch")
    assert_tight(y, want, "sorted small batch")
    assert torch.equal(y, run_sorted(D))
    # x in the sorted order sits behind the counters at the head of the shared workspace: a split-K
    # call on the same stream right after still finds them zero
    L2 = layer(931, 512, 192, bits, 128, False, M=1)
    p2 = _lib.plan_for(_lib.KERNEL_GROUPED, 1, 512, 192, bits, 128, False, split_k=2)
    assert p2.split_k == 2 and p2.workspace_bytes > 0
    assert_close(run_gemm(to_dev(L2, dev), plan=p2), expected_output(L2), "split-K call after a sorted small batch")
    with pytest.raises(_lib.GptqHipError) as e:    # larger batches are not for this entry point
        qs, kmap = pack.sort_channels_by_group(D["qweight"], D["g_idx"], bits, gs)
        x17 = torch.zeros((17, K), dtype=torch.float16, device=dev)
        ops.gemm_sorted(x17, qs, D["qzeros"], D["scales"], kmap, None, bits, gs,
                        plan=_lib.select(17, K, N, bits, gs, False))
    assert e.value.status == _lib.ERR_UNSUPPORTED


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N,gs", [(96, 32, 32), (1024, 416, 32), (2048, 1056, 256), (11008, 256, 128), (1024, 160, -1),
                                    (4096, 352, 128)])
def test_library_sort_equals_the_torch_preparation(dev, bits, K, N, gs):
    # gptq_hip_sort_channels against pack.sort_channels_by_group: both tensors bit for bit
    L = layer(980 + K, K, N, bits, gs, True)
    D = to_dev(L, dev)
    want = pack.sort_channels_by_group(D["qweight"], D["g_idx"], bits, gs)
    if want is None:
        with pytest.raises(_lib.GptqHipError) as e:
            ops.sort_channels(D["qweight"], D["g_idx"], bits, gs)
        assert e.value.status == _lib.ERR_UNSUPPORTED
        return
    got = ops.sort_channels(D["qweight"], D["g_idx"], bits, gs)
    assert torch.equal(got[1], want[1])
    assert torch.equal(got[0], want[0])
    # a contiguous g_idx is its own sorted order
    contiguous = (torch.arange(K, device=dev) // (K if gs == -1 else gs)).to(torch.int32)
    same, kmap = ops.sort_channels(D["qweight"], contiguous, bits, gs)
    assert torch.equal(same, D["qweight"]) and torch.equal(kmap[K:].long(), torch.arange(K, device=dev))


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("M", [1, 2])
@pytest.mark.parametrize("split", [1, 2, 5, 16])
def test_sorted_decode_forced_split_k(dev, bits, M, split):
    # with K split over workgroups each one keeps only the channels whose sorted position is its own
    K, N, gs = 2048, 320, 128
    L = layer(950 + split, K, N, bits, gs, True, M=M, bias=True)
    D = to_dev(L, dev)
    try:
        plan = _lib.plan_for(_lib.KERNEL_GROUPED, M, K, N, bits, gs, False, split_k=split)
    except _lib.GptqHipError as e:
        assert e.status == _lib.ERR_UNSUPPORTED
        pytest.skip("this split is outside the GROUPED family for the shape")
    y = run_sorted(D, plan=plan)
    assert_close(y, expected_output(L), f"sorted split={split}")
    assert_tight(y, expected_output(L), f"sorted split={split}")


def test_sorted_decode_integer_exact_and_rejections(dev):
    # unit scales, zero points 1 (stored 0), integer x: every product and sum is exact in fp32
    K, N, gs, bits = 4096, 352, 128, 3
    L = layer(960, K, N, bits, gs, True, M=1)
    L["scales"] = torch.ones_like(L["scales"])
    L["qzeros"] = torch.zeros_like(L["qzeros"])
    L["x"] = torch.randint(-2, 3, (1, K), generator=torch.Generator().manual_seed(5)).half()
    D = to_dev(L, dev)
    codes = torch.from_numpy(pack.unpack_along_axis0(L["qweight"].numpy(), bits).astype(np.float64))
    want = (L["x"].double() @ (codes - 1.0))
    assert torch.equal(run_sorted(D).cpu().double(), want.half().double())
    # a plan of another family, a map that is not 16-byte aligned, 3-bit groups narrower than 32
    qs, kmap = pack.sort_channels_by_group(D["qweight"], D["g_idx"], bits, gs)
    with pytest.raises(_lib.GptqHipError) as e:
        ops.gemm_sorted(D["x"], qs, D["qzeros"], D["scales"], kmap, None, bits, gs,
                        plan=_lib.select_tiled(1, K, N, bits, gs))
    assert e.value.status == _lib.ERR_UNSUPPORTED
    shifted = torch.zeros(2 * K + 1, dtype=torch.int32, device=dev)[1:]
    shifted.copy_(kmap)
    with pytest.raises(_lib.GptqHipError) as e:
        ops.gemm_sorted(D["x"], qs, D["qzeros"], D["scales"], shifted, None, bits, gs)
    assert e.value.status == _lib.ERR_BAD_ARG


@pytest.mark.parametrize("bits", [3, 4])
def test_quantlinear_decode_uses_the_sorted_copy(dev, bits):
    K, N, gs = 2048, 12288, 128   # wide enough for the decode family to take two rows as well (and for the
    #                               module to prefer the sorted copy over the tiled one at these row counts)
    L = layer(44, K, N, bits, gs, True, M=2, bias=True)
    q = QuantLinear(bits, gs, K, N, True, tile_for_prefill=False)   # (this test is about the sorted copy)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q = q.to(dev)
    assert q._sorted is None
    y = q(L["x"].to(dev))
    assert q._sorted is not None and q._sorted[1] is not None     # built by the first decode-size call
    assert_close(y, expected_output(L), "module decode, sorted")
    assert_close(q(L["x"][:1].to(dev)), expected_output(L)[:1], "module decode, sorted, one row")
    x8 = torch.randn(8, K, generator=torch.Generator().manual_seed(8)).half()
    assert_close(q(x8.to(dev)), expected_output(L, x=x8), "module small batch, sorted")
    # switching the preparation off gives the same numbers from the checkpoint's own tensors
    q.sort_for_decode = False
    assert_tight(q(L["x"].to(dev)), y.cpu(), "module decode, unsorted")
    # new weights invalidate the copy
    q.sort_for_decode = True
    L2 = layer(45, K, N, bits, gs, True, M=2, bias=True)
    q.load_state_dict({k: L2[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    L2["x"] = L["x"]
    assert_close(q(L["x"].to(dev)), expected_output(L2), "module decode after reload")


@pytest.mark.parametrize("bits", [3, 4])
def test_quantlinear_forward(dev, bits):
    K, N, gs = 512, 256, 128
    L = layer(42, K, N, bits, gs, True, M=6, bias=True)
    q = QuantLinear(bits, gs, K, N, True)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q = q.to(dev)
    x = L["x"].reshape(2, 3, K).to(dev)
    y = q(x)
    assert y.shape == (2, 3, N) and y.dtype == torch.float16
    assert_close(y.reshape(6, N), expected_output(L), "module forward")
    y32 = q(x.float())  # any float dtype is accepted and cast to fp16, as the reference does
    assert torch.equal(y32, y)
    w = q.dequantize().cpu()
    assert torch.equal(w.view(torch.int16), expected_weight(L).view(torch.int16))
    # contiguous g_idx is detected and handled by the no-gather path
    q2 = QuantLinear(bits, gs, K, N, False)
    L2 = layer(43, K, N, bits, gs, False, M=1)
    q2.load_state_dict({k: L2[k] for k in ("qweight", "qzeros", "scales", "g_idx")})
    q2 = q2.to(dev)
    assert q2._kernel_g_idx() is None
    assert_close(q2(L2["x"].to(dev)), expected_output(L2), "module forward, contiguous groups")


def test_module_switches_to_dequant_plus_library_gemm_for_long_prompts(dev):
    K, N, gs = 256, 96, 64
    L = layer(78, K, N, 3, gs, True, M=40, bias=True)
    q = QuantLinear(3, gs, K, N, True, kernel_switch_threshold=32)
    q.qweight, q.qzeros, q.scales, q.g_idx, q.bias = L["qweight"], L["qzeros"], L["scales"], L["g_idx"], L["bias"]
    q = q.to(dev)
    y_lib = q(L["x"].to(dev))                 # 40 rows >= 32: library GEMM on the materialised weight
    q.kernel_switch_threshold = None
    y_fused = q(L["x"].to(dev))               # fused kernel
    assert_close(y_lib, expected_output(L), "library path")
    assert_close(y_fused, expected_output(L), "fused path")


def test_module_falls_back_to_dequant_plus_library_gemm_for_uncovered_shapes(dev):
    # activation order with more groups than any fused kernel's LDS table holds
    K, N, gs, M = 36864, 64, 32, 4
    L = layer(77, K, N, 4, gs, True, M=M, bias=True)
    with pytest.raises(_lib.GptqHipError):
        _lib.select(M, K, N, 4, gs, True)
    q = QuantLinear(4, gs, K, N, True)
    q.qweight, q.qzeros, q.scales, q.g_idx, q.bias = L["qweight"], L["qzeros"], L["scales"], L["g_idx"], L["bias"]
    q = q.to(dev)
    y = q(L["x"].to(dev))
    assert_close(y, expected_output(L), "fallback")


def test_bad_g_idx_is_rejected_by_the_module(dev):
    q = QuantLinear(4, 32, 64, 32, False).to(dev)
    q.g_idx[3] = 99
    with pytest.raises(ValueError, match="g_idx"):
        q(torch.zeros(1, 64, device=dev))


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("K,N", [(2048, 4096), (1024, 11008)])
def test_module_forward_replays_in_a_graph(dev, bits, K, N):
    """Decoding loops replay a captured graph: the module's calls (decode kernels, among them the one whose
    halved tiles meet in the slots of a workspace of their own (11008 columns), small batch behind the
    reorder pass, pack pass + matmul + reduce pass) must give the eager result on every replay, with the
    program's own eager work between replays."""
    gs = 128
    L = layer(970 + bits, K, N, bits, gs, True, M=40, bias=True)
    q = QuantLinear(bits, gs, K, N, True)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q = q.to(dev)
    gen = torch.Generator().manual_seed(12)
    xs = {M: torch.randn(M, K, generator=gen).half().to(dev) for M in (1, 4, 8, 40)}
    for M in xs:          # eager first: workspaces and the sorted copy are allocated outside the capture
        q(xs[M])
    torch.cuda.synchronize(dev)
    stream = torch.cuda.Stream(device=dev)
    graph = torch.cuda.CUDAGraph()
    outs = {}
    with torch.cuda.stream(stream):
        for M in xs:
            q(xs[M])      # the side stream gets its own workspace here, before the capture
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            for M in xs:
                outs[M] = q(xs[M])
    for rep in range(3):
        for M in xs:      # new inputs in place, eager reference computed between the replays
            xs[M].copy_(torch.randn(M, K, generator=gen).half())
        want = {M: q(xs[M]).clone() for M in xs}
        torch.cuda.synchronize(dev)
        graph.replay()
        torch.cuda.synchronize(dev)
        for M in xs:
            assert torch.equal(outs[M], want[M]), (rep, M)
            assert_close(outs[M], expected_output(L, x=xs[M].cpu()), f"graph replay {rep}, M={M}")


def test_module_runs_on_two_streams_at_once(dev):
    """Two host streams run the same layers back to back without waiting for each other: every (device, stream)
    has workspaces of its own (also the one whose exchange slots the halved tiles of 11008 columns use), so the
    results equal those of one stream alone."""
    K, gs = 1024, 128
    layers = []
    for i, (bits, N) in enumerate(((4, 11008), (3, 11008), (4, 4096))):
        L = layer(1200 + i, K, N, bits, gs, True, M=40, bias=True)
        q = QuantLinear(bits, gs, K, N, True)
        q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
        layers.append((L, q.to(dev)))
    gen = torch.Generator().manual_seed(5)
    xs = {M: torch.randn(M, K, generator=gen).half().to(dev) for M in (1, 4, 40)}
    want = {(i, M): q(x).clone() for i, (L, q) in enumerate(layers) for M, x in xs.items()}
    torch.cuda.synchronize(dev)
    streams = [torch.cuda.Stream(device=dev) for _ in range(2)]
    got = [{}, {}]
    for rep in range(6):
        for si, st in enumerate(streams):
            with torch.cuda.stream(st):
                for i, (L, q) in enumerate(layers):
                    for M, x in xs.items():
                        got[si][(i, M, rep)] = q(x)
    torch.cuda.synchronize(dev)
    for si in range(2):
        for (i, M, rep), y in got[si].items():
            assert torch.equal(y, want[(i, M)]), (si, i, M, rep)
    for i, (L, q) in enumerate(layers):
        for M, x in xs.items():
            assert_close(want[(i, M)], expected_output(L, x=x.cpu()), f"layer {i}, M={M}")


def test_torch_operator_equals_the_python_front_end(dev):
    L = layer(990, 512, 256, 3, 128, True, M=5, bias=True)
    D = to_dev(L, dev)
    a = torch.ops.gptq_hip.gemm(D["x"], D["qweight"], D["qzeros"], D["scales"], D["g_idx"], D["bias"], 3, 128)
    assert torch.equal(a, run_gemm(D))
    w = torch.ops.gptq_hip.dequant(D["qweight"], D["qzeros"], D["scales"], D["g_idx"], 3, 128)
    assert torch.equal(w.cpu().view(torch.int16), expected_weight(L).view(torch.int16))
    # the operators are the C++ ones of csrc/binding.cpp (built beside the kernel library), and each gives what
    # the ctypes front end gives on the same tensors
    assert ops.NATIVE_OPS
    qs, kmap = ops.sort_channels(D["qweight"], D["g_idx"], 3, 128)
    b = torch.ops.gptq_hip.gemm_sorted(D["x"], qs, D["qzeros"], D["scales"], kmap, D["bias"], 3, 128)
    assert torch.equal(b, ops.gemm_sorted(D["x"], qs, D["qzeros"], D["scales"], kmap, D["bias"], 3, 128))
    qtile, sz, xsrc, kinv = ops.tile_prepare(D["qweight"], D["qzeros"], D["scales"], D["g_idx"], 3, 128)
    for M in (5, 3):
        c = torch.ops.gptq_hip.gemm_tiled(D["x"][:M], qtile, sz, xsrc, kinv, D["bias"], 3, 128)
        assert torch.equal(c, ops.gemm_tiled(D["x"][:M], qtile, sz, xsrc, kinv, D["bias"], 3, 128))
    assert_close(a, expected_output(L), "C++ operator")
    # a layer's tensors bound once (what QuantLinear calls): first call checked, later calls on the kept plan
    for kind, args in ((0, (D["qweight"], D["qzeros"], D["scales"], D["g_idx"], None)),
                       (1, (qs, D["qzeros"], D["scales"], kmap, None)), (2, (qtile, sz, None, xsrc, kinv))):
        bound = torch.classes.gptq_hip.Layer(kind, *args, D["bias"], 3, 128)
        for x in (D["x"], D["x"], D["x"][:2], D["x"]):
            assert_close(bound.forward(x), expected_output(L)[: x.shape[0]], f"bound layer, kind {kind}")
        with pytest.raises(RuntimeError, match="no CPU fallback"):
            bound.forward(D["x"].cpu())
        with pytest.raises(RuntimeError):
            bound.forward(D["x"][:, :256].contiguous())
    with pytest.raises(RuntimeError, match="must be"):
        torch.ops.gptq_hip.gemm(D["x"].float(), D["qweight"], D["qzeros"], D["scales"], D["g_idx"], D["bias"], 3, 128)
    with pytest.raises(RuntimeError, match="UNSUPPORTED|unsupported|not supported|status"):
        torch.ops.gptq_hip.gemm_tiled(D["x"], qtile, sz, xsrc, kinv, D["bias"], 3, 16)
