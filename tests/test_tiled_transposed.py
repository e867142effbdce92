"""GPU parity of the transposed product gx = gy @ W^T (the gradient of y = x @ W with respect to x; the reference's
transpose_matmul248, auto_gptq/nn_modules/qlinear_triton.py:195-273,298-317): the library's preparation against
the torch statement of the copy, and gptq_hip_gemm_tiled_transposed (through the C ABI) against the CPU oracle's
dequantised weight on the same seeded inputs.  The kernel forms the reference's rounded fp16 weights and adds in
fp32, so the tight bound applies as well as the contract's rtol = atol = 1e-2."""
import ctypes

import pytest
import torch

from autogptq.tvm_amd import _lib, ops, pack
from autogptq.tvm_amd.qlinear import QuantLinear
from tests.parity_util import assert_close, assert_tight, expected_weight, layer, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def prepare(D):
    """(qtile_t, szt, xsrc): the forward preparation gives the map, the transposed one the copy."""
    act = D["desc_act"]
    xsrc = ops.tile_prepare(D["qweight"], D["qzeros"], D["scales"], D["g_idx"] if act else None, D["bits"],
                            D["group_size"])[2] if act else None
    qtile_t, szt = ops.tile_prepare_transposed(D["qweight"], D["qzeros"], D["scales"], xsrc, D["bits"], D["group_size"])
    return qtile_t, szt, xsrc


def grad_rows(seed, M, N):
    return torch.randn(M, N, generator=torch.Generator().manual_seed(seed)).half()


def run_t(D, prep, gy, plan=None):
    qtile_t, szt, xsrc = prep
    return ops.gemm_tiled_transposed(gy, qtile_t, szt, xsrc, D["K"], D["bits"], D["group_size"], plan=plan)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(64, 32, 32), (96, 96, 32), (1024, 416, 32), (2048, 1056, 256), (1024, 160, -1),
                                    (4096, 352, 128)])
@pytest.mark.parametrize("desc_act", [False, True])
def test_library_preparation_equals_the_torch_statement(dev, bits, K, N, gs, desc_act):
    L = layer(3100 + K, K, N, bits, gs, desc_act)
    D = to_dev(L, dev)
    g = D["g_idx"] if desc_act else None
    want = pack.tile_layout_transposed(D["qweight"], D["qzeros"], D["scales"], g, bits, gs)
    got = prepare(D)
    assert torch.equal(got[0], want[0]), "qtile_t"
    assert torch.equal(got[1], want[1]), "szt"


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(32, 32, 32), (96, 96, 32), (160, 96, -1), (384, 64, 64), (1024, 416, 32),
                                    (2048, 1056, 256), (4096, 352, 128), (352, 4096, 32)])
@pytest.mark.parametrize("M", [1, 7, 40, 130])
def test_transposed_product_shapes(dev, bits, K, N, gs, M):
    # N that is not a multiple of 64 (a padded last block of the reduction), an odd number of position tiles,
    # every tile height, group sizes from one tile to the whole layer, with and without an activation order
    for desc_act in (False, True):
        L = layer(3200 + K + N, K, N, bits, gs, desc_act)
        D = to_dev(L, dev)
        prep = prepare(D)
        gy = grad_rows(3300 + M, M, N)
        gx = run_t(D, prep, gy.to(dev))
        assert gx.shape == (M, K) and gx.dtype == torch.float16
        want = gy.float() @ expected_weight(L).float().t()
        what = f"transposed bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}"
        assert_close(gx, want, what)
        assert_tight(gx, want, what)
        assert torch.equal(gx, run_t(D, prep, gy.to(dev))), "two identical calls differ"


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("M,row_tiles", [(40, 1), (40, 2), (64, 2), (65, 4), (130, 1), (130, 2), (130, 4), (257, 4)])
def test_transposed_every_block_height_on_a_narrow_layer(dev, bits, M, row_tiles):
    # the planner gives narrow layers shorter row blocks than wide ones: every height the kernel is built for, forced
    K, N, gs = 416, 1024, 32
    L = layer(3450 + M, K, N, bits, gs, True)
    D = to_dev(L, dev)
    plan = _lib.select_tiled_transposed(M, K, N, bits, gs)
    plan.row_tiles = row_tiles
    plan.m_blocks = plan.grid_z = -(-M // (32 * row_tiles))
    plan.split_k = plan.grid_y = 1
    plan.k_chunk = -(-(N // 64) // plan.waves_k)
    plan.lds_bytes = max(plan.waves_k * row_tiles * 2 * 4096, 2 * plan.waves_k * plan.k_chunk * 256)
    plan.workspace_bytes = 16384 + plan.waves_k * plan.k_chunk * 4 * row_tiles * plan.m_blocks * 1024
    prep = prepare(D)
    gy = grad_rows(3460 + M, M, N)
    g1 = run_t(D, prep, gy.to(dev), plan=plan)
    want = gy.float() @ expected_weight(L).float().t()
    assert_close(g1, want, f"transposed M={M} row_tiles={row_tiles}")
    assert_tight(g1, want, f"transposed M={M} row_tiles={row_tiles}")
    assert torch.equal(g1, run_t(D, prep, gy.to(dev), plan=plan))


@pytest.mark.parametrize("bits", [3, 4, 8])
@pytest.mark.parametrize("split", [1, 2, 3, 5])
@pytest.mark.parametrize("M", [20, 130])
def test_transposed_forced_split(dev, bits, split, M):
    K, N, gs = 352, 4096, 32
    L = layer(3400 + split, K, N, bits, gs, True)
    D = to_dev(L, dev)
    plan = _lib.select_tiled_transposed(M, K, N, bits, gs)
    blocks = N // 64
    plan.split_k, plan.grid_y = split, split
    plan.k_chunk = -(-blocks // (plan.waves_k * split))
    part = (split * M * K * 4 + 255) // 256 * 256 if split > 1 else 0
    plan.lds_bytes = max(plan.waves_k * plan.row_tiles * 2 * 4096, 2 * plan.waves_k * plan.k_chunk * 256)
    plan.workspace_bytes = 16384 + part + split * plan.waves_k * plan.k_chunk * 4 * plan.row_tiles * plan.m_blocks * 1024
    prep = prepare(D)
    gy = grad_rows(3500 + M, M, N)
    g1 = run_t(D, prep, gy.to(dev), plan=plan)
    g2 = run_t(D, prep, gy.to(dev), plan=plan)
    want = gy.float() @ expected_weight(L).float().t()
    assert_close(g1, want, f"transposed split={split}")
    assert_tight(g1, want, f"transposed split={split}")
    assert torch.equal(g1, g2)


def test_transposed_integer_exact_guard_bands_and_rejections(dev):
    # gy = 1, scales = 1, one group: gx[k] = sum_n (q - z), an integer below 2048
    for bits in (2, 3, 4):
        L = layer(3600, 64, 96, bits, -1, False)
        L["scales"] = torch.ones_like(L["scales"])
        D = to_dev(L, dev)
        gx = run_t(D, prepare(D), torch.ones((2, 96), dtype=torch.float16, device=dev)).float().cpu()
        want = (L["codes"].float() - L["zeros"][0].float()[None, :]).sum(dim=1)
        assert torch.equal(gx[0], want) and torch.equal(gx[1], want)
    M, K, N = 37, 512, 96
    L = layer(3601, K, N, 4, 128, True)
    D = to_dev(L, dev)
    qtile_t, szt, xsrc = prepare(D)
    gy = grad_rows(3602, M, N)
    guard = 4096
    buf = torch.full((guard + M * K + guard,), 1234.0, dtype=torch.float16, device=dev)
    out = buf[guard: guard + M * K].view(M, K)
    ops.gemm_tiled_transposed(gy.to(dev), qtile_t, szt, xsrc, K, 4, 128, out=out)
    assert_close(out, gy.float() @ expected_weight(L).float().t(), "guarded out")
    assert bool((buf[:guard] == 1234.0).all()) and bool((buf[guard + M * K:] == 1234.0).all())
    lib = _lib.lib()
    fake, null = ctypes.c_void_p(0x1000), ctypes.c_void_p(None)
    assert lib.gptq_hip_gemm_tiled_transposed(fake, fake, fake, null, fake, null, 0, 40, 4096, 352, 4, 128, None, null) == _lib.ERR_WORKSPACE
    assert lib.gptq_hip_gemm_tiled_transposed(fake, fake, fake, null, fake, fake, 1 << 24, 8, 4096, 352, 4, 16, None, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_gemm_tiled_transposed(fake, fake, fake, null, null, fake, 1 << 24, 8, 4096, 352, 4, 128, None, null) == _lib.ERR_BAD_ARG
    p = _lib.select_tiled(17, 4096, 352, 4, 128)   # a plan of the forward product (matmul kernel): its grid is not this product's
    assert lib.gptq_hip_gemm_tiled_transposed(fake, fake, fake, null, fake, fake, 1 << 24, 8, 4096, 352, 4, 128, ctypes.byref(p),
                                              null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_tile_prepare_transposed(fake, fake, fake, null, null, fake, 4096, 352, 4, 128, null) == _lib.ERR_BAD_ARG
    other = ctypes.c_void_p(0x2000)
    assert lib.gptq_hip_tile_prepare_transposed(fake, fake, fake, null, other, fake, 4096, 352, 4, 16, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_tile_prepare_transposed(fake, fake, fake, null, fake, fake, 4096, 352, 4, 128, null) == _lib.ERR_BAD_ARG  # in place
    assert lib.gptq_hip_tiled_transposed_bytes(4096, 352, 3) == 4096 * 384 * 3 // 8
    assert lib.gptq_hip_tiled_transposed_table_bytes(4096, 352, 128) == 32 * 6 * 256


FULL = [
    ("c4-int4-4096x11008-act", 4, 4096, 11008, 128, True, [16, 128, 256]),
    ("c4-int3-4096x11008-act", 3, 4096, 11008, 128, True, [64, 128]),
    ("c4-int4-11008x4096-act", 4, 11008, 4096, 128, True, [128]),
    ("c3-int4-4096x4096", 4, 4096, 4096, 128, False, [8, 1024]),
    ("int4-4096x4096-act", 4, 4096, 4096, 128, True, [64, 128, 256]),       # (a narrow layer: shorter row blocks)
    ("int3-9216x18432-act", 3, 9216, 18432, 128, True, [128]),             # (the reduction in ranges over two turns)
    ("int8-4096x11008-act", 8, 4096, 11008, 128, True, [128]),
    ("int2-11008x4096", 2, 11008, 4096, 128, False, [64]),
    ("c5-int3-9216x36864-act-g1", 3, 9216, 36864, -1, True, [32]),
    ("int4-352x65536-act", 4, 352, 65536, 32, True, [40]),   # a reduction longer than one workgroup's table
]


@pytest.mark.parametrize("name,bits,K,N,gs,desc_act,Ms", FULL, ids=[f[0] for f in FULL])
def test_transposed_full_size(dev, name, bits, K, N, gs, desc_act, Ms):
    L = layer(7400 + [f[0] for f in FULL].index(name), K, N, bits, gs, desc_act)
    D = to_dev(L, dev)
    wt = expected_weight(L).float().t().contiguous()
    prep = prepare(D)
    for M in Ms:
        gy = grad_rows(7500 + M, M, N)
        gx = run_t(D, prep, gy.to(dev))
        want = gy.float() @ wt
        assert_close(gx, want, f"transposed {name} M={M}")
        assert_tight(gx, want, f"transposed {name} M={M}")


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("desc_act", [False, True])
def test_module_gradient_runs_fused(dev, bits, desc_act):
    """The gradient for x below the switch to the library GEMM is the fused transposed product; above it (and with
    the tiled copies switched off) W from the dequant kernel and the library GEMM: the same numbers to the tight
    bound."""
    K, N, gs, M = 512, 416, 128, 24
    L = layer(3700 + bits, K, N, bits, gs, desc_act, M=M, bias=True)
    q = QuantLinear(bits, gs, K, N, True, kernel_switch_threshold=64)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q = q.to(dev)
    gy = grad_rows(3710, M, N)
    want = gy.float() @ expected_weight(L).float().t()
    x = L["x"].to(dev).requires_grad_(True)
    q(x).backward(gy.to(dev))
    assert q._tiled_t is not None and q._tiled_t[1] is not None
    assert_close(x.grad, want, "fused gradient")
    assert_tight(x.grad, want, "fused gradient")
    # three leading dimensions, a float32 gradient
    g3 = q.grad_input(gy.float().to(dev).view(2, 3, 4, N))
    assert g3.shape == (2, 3, 4, K)
    assert_tight(g3.reshape(M, K), want, "fused gradient, 4-D")
    # the library route: long batches, or no tiled copies
    big = grad_rows(3711, 64, N)
    assert_tight(q.grad_input(big.to(dev)), big.float() @ expected_weight(L).float().t(), "library gradient")
    off = QuantLinear(bits, gs, K, N, True, tile_for_prefill=False)
    off.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    off = off.to(dev)
    assert_tight(off.grad_input(gy.to(dev)), want, "gradient without the tiled copies")
    assert off._tiled_t is None
    # a compact layer keeps the copy it had
    assert q.compact() and q.prepare_transposed() is not None
    assert_tight(q.grad_input(gy.to(dev)), want, "compact layer, fused gradient")
    # new weights invalidate the copy
    q2 = QuantLinear(bits, gs, K, N, True)
    q2.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    q2 = q2.to(dev)
    q2.grad_input(gy.to(dev))
    L2 = layer(3720 + bits, K, N, bits, gs, desc_act, bias=True)
    q2.load_state_dict({k: L2[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    assert_tight(q2.grad_input(gy.to(dev)), gy.float() @ expected_weight(L2).float().t(), "gradient after reload")
