"""GPU parity of the TILED family: the library's preparation against the torch statement of the format, and
gptq_hip_gemm_tiled (through the C ABI) against the CPU oracle on the same seeded inputs.  The kernel forms the
reference's rounded fp16 weights, so the tight bound applies as well as the contract's rtol = atol = 1e-2."""
import ctypes

import pytest
import torch

from autogptq.tvm_amd import _lib, ops, pack
from autogptq.tvm_amd.qlinear import QuantLinear
from tests.parity_util import assert_close, assert_tight, expected_output, expected_weight, layer, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda:0")


def prepare(D):
    g = D["g_idx"] if D["desc_act"] else None
    return ops.tile_prepare(D["qweight"], D["qzeros"], D["scales"], g, D["bits"], D["group_size"])


def tile_decode_plan(M, K, N, bits, gs):
    """The plan of the workgroup-per-tile decode kernel (the family's choice when x does not fit the LDS of the
    one-workgroup-per-CU kernel), made by hand so that both kernels are tested on every shape."""
    plan = _lib.select_tiled(M, K, N, bits, gs, decode=True)
    return tile_decode_plan_of(plan, M, K, N, bits, gs)   # (a workgroup per whole tile, whatever the family halves)


def tile_decode_plan_of(plan, M, K, N, bits, gs):
    g = K if gs == -1 else gs
    mr = 1 if M <= 1 else (2 if M <= 2 else 4)
    tiles, S_total = N // 32, -(-K // 64)
    kw = 4 if tiles * 4 >= 1024 else (8 if tiles * 8 >= 1024 else 16)
    while kw > 4 and kw > S_total:
        kw >>= 1
    steps = -(-S_total // kw)
    span = steps * kw * 64
    groups = min((span - 1) // g + 2, K // g)
    plan.waves_n, plan.waves_k, plan.split_k, plan.k_chunk = 1, kw, 1, steps
    plan.grid_x, plan.grid_y, plan.grid_z, plan.block = tiles, 1, 1, 64 * kw
    plan.lds_bytes = mr * span * 2 + 64 + (span // 32) * mr * 8 + groups * 128 + kw * mr * 128
    plan.workspace_bytes, plan.flags = 0, 0    # (whole tiles: no slots, whatever the family's own plan needs)
    return plan


def cu_decode_plan(M, K, N, bits, gs, grid=None):
    """The plan of the one-workgroup-per-CU decode kernel (16-column units), whatever the family would choose;
    ``grid`` workgroups (default: one per unit up to 256).  None when x and the tables do not fit LDS."""
    plan = _lib.select_tiled(M, K, N, bits, gs, decode=True)
    g = K if gs == -1 else gs
    units = N // 16
    grid = grid or min(units, 256)
    upw = -(-units // grid)
    mr = 1 if M <= 1 else (2 if M <= 2 else 4)
    V = -(-(-(-K // 64)) // 2)
    span = V * 128
    lds = mr * span * 2 + 64 + span // 32 * mr * 8 + upw * (K // g) * 128 + upw * 16 * mr * 256
    if lds > 150 * 1024:
        return None
    plan.row_tiles, plan.waves_n, plan.waves_k, plan.split_k, plan.k_chunk = mr, 2, 16, 1, -(-V // 16)
    plan.grid_x, plan.grid_y, plan.grid_z, plan.block, plan.lds_bytes, plan.workspace_bytes = grid, 1, 1, 1024, lds, 0
    plan.flags = 0
    return plan


def unrounded_output(L, x):
    """x @ (scale * (q - zero)) (+ bias) in fp64 with the weights NOT rounded to fp16."""
    import numpy as np

    from oracle import gptq_oracle

    bits = L["bits"]
    q = gptq_oracle.unpack_bitstream(L["qweight"].numpy(), bits, axis=0).astype(np.float64)
    z = (gptq_oracle.unpack_bitstream(L["qzeros"].numpy(), bits, axis=1) + 1).astype(np.float64)
    g = L["g_idx"].numpy().astype(np.int64)
    w = L["scales"].numpy().astype(np.float64)[g] * (q - z[g])
    y = x.numpy().astype(np.float64) @ w
    if L.get("bias") is not None:
        y = y + L["bias"].numpy().astype(np.float64)
    return torch.from_numpy(y)


def run_tiled(D, prep, x=None, plan=None):
    qtile, sz, xsrc, kinv = prep
    act = D["desc_act"]
    return ops.gemm_tiled(D["x"] if x is None else x, qtile, sz, xsrc if act else None, kinv if act else None,
                          D.get("bias"), D["bits"], D["group_size"], plan=plan)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(64, 32, 32), (96, 32, 32), (1024, 416, 32), (2048, 1056, 256), (11008, 256, 128),
                                    (1024, 160, -1), (4096, 352, 128)])
@pytest.mark.parametrize("desc_act", [False, True])
def test_library_preparation_equals_the_torch_statement(dev, bits, K, N, gs, desc_act):
    L = layer(1100 + K, K, N, bits, gs, desc_act)
    D = to_dev(L, dev)
    g = D["g_idx"] if desc_act else None
    want = pack.tile_layout(D["qweight"], D["qzeros"], D["scales"], g, bits, gs)
    got = ops.tile_prepare(D["qweight"], D["qzeros"], D["scales"], g, bits, gs)
    for a, b, what in zip(got, want, ("qtile", "sz", "xsrc", "kinv")):
        assert torch.equal(a, b), what
    # an explicit contiguous g_idx is its own sorted order
    if not desc_act:
        again = ops.tile_prepare(D["qweight"], D["qzeros"], D["scales"], D["g_idx"], bits, gs)
        for a, b in zip(again, want):
            assert torch.equal(a, b)


M_EDGES = [1, 2, 5, 16, 17, 31, 32, 33, 64, 65, 127, 128, 129, 257]


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("desc_act", [False, True])
@pytest.mark.parametrize("M", M_EDGES)
def test_tiled_ragged_m(dev, bits, desc_act, M):
    L = layer(1200 + M, 512, 192, bits, 128, desc_act, M=M, bias=(M % 2 == 1))
    D = to_dev(L, dev)
    y = run_tiled(D, prepare(D))
    assert y.shape == (M, 192) and y.dtype == torch.float16
    assert_close(y, expected_output(L), f"tiled bits={bits} act={desc_act} M={M}")
    assert_tight(y, expected_output(L), f"tiled bits={bits} act={desc_act} M={M}")


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(32, 32, 32), (96, 32, 32), (160, 96, -1), (384, 64, 64), (1024, 416, 32),
                                    (2048, 1056, 256), (4096, 352, 128)])
@pytest.mark.parametrize("M", [1, 7, 40, 130])
def test_tiled_odd_shapes(dev, bits, K, N, gs, M):
    # K that is not a multiple of 64 (a padded last block), an odd number of column tiles, every tile height
    for desc_act in (False, True):
        L = layer(1300 + K + N, K, N, bits, gs, desc_act, M=M, bias=True)
        D = to_dev(L, dev)
        prep = prepare(D)
        y = run_tiled(D, prep)
        assert_close(y, expected_output(L), f"tiled bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
        assert_tight(y, expected_output(L), f"tiled bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
        assert torch.equal(y, run_tiled(D, prep)), "two identical calls differ"


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(1024, 416, 128), (4096, 352, 64), (2048, 11008, 128)])
def test_tiled_small_batches_read_x_without_the_pack_pass(dev, bits, K, N, gs):
    # 5 to 16 rows of a layer without an activation order: the matmul kernel reads its fragments from x itself.
    # Handing the same layer over with its (identity) channel maps forces the pack pass: same fragments, so the
    # two results are the same bits.
    L = layer(2500 + bits, K, N, bits, gs, False, M=16, bias=True)
    D = to_dev(L, dev)
    qtile, sz, xsrc, kinv = prepare(D)
    w16 = expected_weight(L)
    for M in (5, 9, 16):
        x = L["x"][:M].contiguous()
        direct = ops.gemm_tiled(x.to(dev), qtile, sz, None, None, D["bias"], bits, gs)
        packed = ops.gemm_tiled(x.to(dev), qtile, sz, xsrc, kinv, D["bias"], bits, gs)
        want = expected_output(L, x=x, w16=w16)
        assert_close(direct, want, f"direct M={M}")
        assert_tight(direct, want, f"direct M={M}")
        assert torch.equal(direct, packed), f"M={M}: reading x directly and through the pack pass differ"


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("split", [1, 2, 3, 5])
@pytest.mark.parametrize("M", [20, 130])
def test_tiled_forced_split_k(dev, bits, split, M):
    K, N, gs = 4096, 352, 128
    L = layer(1400 + split, K, N, bits, gs, True, M=M, bias=True)
    D = to_dev(L, dev)
    plan = _lib.select_tiled(M, K, N, bits, gs)
    blocks = K // 64
    plan.split_k, plan.grid_y = split, split
    plan.k_chunk = -(-blocks // (plan.waves_k * split))
    part = (split * M * N * 4 + 255) // 256 * 256 if split > 1 else 0
    plan.workspace_bytes = 16384 + part + split * plan.waves_k * plan.k_chunk * 4 * plan.row_tiles * plan.m_blocks * 1024
    prep = prepare(D)
    y1 = run_tiled(D, prep, plan=plan)
    y2 = run_tiled(D, prep, plan=plan)
    assert_close(y1, expected_output(L), f"tiled split={split}")
    assert_tight(y1, expected_output(L), f"tiled split={split}")
    assert torch.equal(y1, y2)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("M,row_tiles", [(33, 2), (64, 2), (65, 4), (127, 4), (130, 4), (257, 4), (40, 1), (130, 2), (257, 1)])
@pytest.mark.parametrize("split", [1, 2])
def test_tiled_every_block_height_on_a_narrow_layer(dev, bits, M, row_tiles, split):
    # the planner gives narrow layers shorter row blocks than wide ones: every height the kernel is built for, forced on
    # one narrow layer (the tall blocks as wide layers get them, and more, shorter blocks than the planner would choose)
    K, N, gs = 1024, 416, 128
    L = layer(1450 + M, K, N, bits, gs, True, M=M, bias=True)
    D = to_dev(L, dev)
    plan = _lib.select_tiled(M, K, N, bits, gs)
    assert plan.kernel == _lib.KERNEL_TILED and plan.waves_n == 1
    blocks = K // 64
    plan.row_tiles = row_tiles
    plan.m_blocks = plan.grid_z = -(-M // (32 * row_tiles))
    plan.lds_bytes = plan.waves_k * row_tiles * 2 * 4096
    plan.split_k, plan.grid_y = split, split
    plan.k_chunk = -(-blocks // (plan.waves_k * split))
    part = (split * M * N * 4 + 255) // 256 * 256 if split > 1 else 0
    plan.workspace_bytes = 16384 + part + split * plan.waves_k * plan.k_chunk * 4 * plan.row_tiles * plan.m_blocks * 1024
    prep = prepare(D)
    y1 = run_tiled(D, prep, plan=plan)
    assert_close(y1, expected_output(L), f"tiled M={M} row_tiles={row_tiles} split={split}")
    assert_tight(y1, expected_output(L), f"tiled M={M} row_tiles={row_tiles} split={split}")
    assert torch.equal(y1, run_tiled(D, prep, plan=plan)), "two identical calls differ"


def test_tiled_integer_exact_and_guard_bands(dev):
    # x = 1, scales = 1, one group: y[n] = sum_k (q - z), an integer (8-bit sums pass 2048: one fp16 rounding)
    for bits in (2, 3, 4, 8):
        L = layer(1500, 64, 64, bits, -1, False, M=2)
        L["scales"] = torch.ones_like(L["scales"])
        L["x"] = torch.ones_like(L["x"])
        D = to_dev(L, dev)
        y = run_tiled(D, prepare(D)).float().cpu()
        want = (L["codes"].float() - L["zeros"][0].float()[None, :]).sum(dim=0).half().float()
        assert torch.equal(y[0], want) and torch.equal(y[1], want)
    M, K, N = 37, 512, 96
    L = layer(1501, K, N, 4, 128, True, M=M)
    D = to_dev(L, dev)
    qtile, sz, xsrc, kinv = prepare(D)
    guard = 4096
    buf = torch.full((guard + M * N + guard,), 1234.0, dtype=torch.float16, device=dev)
    out = buf[guard: guard + M * N].view(M, N)
    ops.gemm_tiled(D["x"], qtile, sz, xsrc, kinv, None, 4, 128, out=out)
    assert_close(out, expected_output(L), "guarded out")
    assert bool((buf[:guard] == 1234.0).all()) and bool((buf[guard + M * N:] == 1234.0).all())


def test_tiled_rejections(dev):
    lib = _lib.lib()
    with pytest.raises(_lib.GptqHipError):       # the decode kernel takes up to eight rows
        _lib.select_tiled(9, 4096, 352, 4, 128, decode=True)
    fake, null = ctypes.c_void_p(0x1000), ctypes.c_void_p(None)
    # no workspace; groups that are not whole 32-channel lane blocks; a plan of another family
    assert lib.gptq_hip_gemm_tiled(fake, fake, fake, null, null, null, fake, null, 0, 40, 4096, 352, 4, 128, None, null) == _lib.ERR_WORKSPACE
    assert lib.gptq_hip_gemm_tiled(fake, fake, fake, null, null, null, fake, fake, 1 << 24, 8, 4096, 352, 4, 16, None, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_gemm_tiled(fake, fake, fake, fake, null, null, fake, fake, 1 << 24, 8, 4096, 352, 4, 128, None, null) == _lib.ERR_BAD_ARG   # a map without its inverse
    p = _lib.select(8, 4096, 352, 4, 128, False)
    assert lib.gptq_hip_gemm_tiled(fake, fake, fake, null, null, null, fake, fake, 1 << 24, 8, 4096, 352, 4, 128, ctypes.byref(p),
                                   null) == _lib.ERR_UNSUPPORTED
    # halved tiles without the flag that asks for a workspace of their own, and the flag on a plan that writes partial sums
    h = _lib.select_tiled(1, 4096, 352, 4, 128)
    assert h.grid_x == 2 * (352 // 32) and h.flags & _lib.PLAN_PRIVATE_ZERO_WORKSPACE
    h.flags = 0
    assert lib.gptq_hip_gemm_tiled(fake, fake, fake, null, null, null, fake, fake, 1 << 24, 1, 4096, 352, 4, 128, ctypes.byref(h),
                                   null) == _lib.ERR_BAD_ARG
    w = tile_decode_plan(1, 4096, 352, 4, 128)
    w.split_k = w.grid_y = 2
    w.k_chunk = -(-(4096 // 64) // (2 * w.waves_k))
    w.workspace_bytes, w.flags = 16384 + 2 * 352 * 4, _lib.PLAN_PRIVATE_ZERO_WORKSPACE
    assert lib.gptq_hip_gemm_tiled(fake, fake, fake, null, null, null, fake, fake, 1 << 24, 1, 4096, 352, 4, 128, ctypes.byref(w),
                                   null) == _lib.ERR_BAD_ARG
    other = ctypes.c_void_p(0x2000)
    assert lib.gptq_hip_tile_prepare(fake, fake, fake, null, other, fake, fake, fake, 4096, 352, 4, 16, null) == _lib.ERR_UNSUPPORTED
    assert lib.gptq_hip_tile_prepare(fake, fake, fake, null, null, fake, fake, fake, 4096, 352, 4, 128, null) == _lib.ERR_BAD_ARG
    assert lib.gptq_hip_tile_prepare(fake, fake, fake, null, fake, fake, fake, fake, 4096, 352, 4, 128, null) == _lib.ERR_BAD_ARG  # in place
    assert lib.gptq_hip_tiled_bytes(4096, 11008, 3) == 4096 * 11008 * 3 // 8
    assert lib.gptq_hip_tiled_bytes(96, 32, 4) == 128 * 32 // 2


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(32, 32, 32), (96, 32, 32), (160, 96, -1), (384, 64, 64), (1024, 416, 32),
                                    (2048, 1056, 256), (4096, 352, 128), (11008, 256, 128), (4096, 64, 64)])
@pytest.mark.parametrize("M", [1, 2, 3, 4])
def test_tiled_decode_rows_and_shapes(dev, bits, K, N, gs, M):
    """The decode kernel of the tiled format (M <= 4): every row count, K that is not a multiple of 64, one
    and many column tiles, group sizes from one lane block to the whole layer, with and without an activation
    order; against the oracle and against the unprepared kernels on the same inputs."""
    for desc_act in (False, True):
        L = layer(1600 + K + M, K, N, bits, gs, desc_act, M=M, bias=(M % 2 == 0))
        D = to_dev(L, dev)
        own = _lib.select_tiled(M, K, N, bits, gs)   # the family's own choice: a decode kernel up to four rows
        assert own.kernel == _lib.KERNEL_TILED_DECODE and own.row_tiles in (1, 2, 4) and own.row_tiles >= M
        prep = prepare(D)
        want = expected_output(L)
        g = D["g_idx"] if desc_act else None
        # (the kernels on the checkpoint layout cover 3 and 4 bits)
        plain = (ops.gemm(D["x"], D["qweight"], D["qzeros"], D["scales"], g, D.get("bias"), bits, gs).cpu()
                 if bits in ops.FUSED_BITS else None)
        # both decode kernels, and the one-workgroup-per-CU kernel on fewer workgroups (several units each)
        plans = [("own", own), ("tile", tile_decode_plan(M, K, N, bits, gs)), ("cu", cu_decode_plan(M, K, N, bits, gs)),
                 ("cu, few workgroups", cu_decode_plan(M, K, N, bits, gs, grid=max(1, (N // 16) // 5)))]
        for what, plan in plans:
            if plan is None:
                continue
            y = run_tiled(D, prep, plan=plan)
            assert_close(y, want, f"decode ({what}) bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
            assert_tight(y, want, f"decode ({what}) bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
            assert torch.equal(y, run_tiled(D, prep, plan=plan)), "two identical calls differ"
            if plain is not None:
                assert_tight(y, plain, "decode vs the unprepared kernels")


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("M", [1, 4])
def test_tiled_decode_split_k(dev, bits, M):
    # a forced split of K over workgroups (what a long K with many rows needs): partial sums and the reduce pass
    K, N, gs = 4096, 352, 128
    L = layer(1700 + M, K, N, bits, gs, True, M=M, bias=True)
    D = to_dev(L, dev)
    prep = prepare(D)
    plan = tile_decode_plan(M, K, N, bits, gs)
    for split in (2, 4):           # two blocks per wave (paired epilogue) and one (the one-block epilogue)
        plan.split_k = plan.grid_y = split
        plan.k_chunk = -(-(K // 64) // (split * plan.waves_k))
        plan.workspace_bytes = 16384 + split * M * N * 4
        y = run_tiled(D, prep, plan=plan)
        assert_close(y, expected_output(L), f"decode split={split}")
        assert_tight(y, expected_output(L), f"decode split={split}")
        assert torch.equal(y, run_tiled(D, prep, plan=plan))


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(1024, 8224, 128), (1024, 11008, 128), (1280, 12288, 128), (2048, 9600, 64),
                                    (2048, 12288, -1), (640, 18368, 128), (1152, 9216, 32),
                                    (8192, 1056, 128), (8256, 512, 64), (8192, 4096, 1024), (9248, 96, 32),
                                    (4096, 4096, 128), (4160, 352, 32), (5120, 2048, 128), (4096, 96, 64)])
@pytest.mark.parametrize("desc_act", [False, True])
def test_tiled_decode_halved_tiles(dev, bits, K, N, gs, desc_act):
    # Up to 128 column tiles past a whole number per CU (256), or every tile of a layer of up to 4096 columns with 4096
    # channels or more (the last eight shapes): the family's plan runs them as two halves along K (equal, or the first one larger:
    # 1280, 1152, 8256 and 9248 channels) that meet through the exchange slots of a workspace of their own; the
    # slots are zero again after every call, so the same workspace serves every row count in turn
    L = layer(8100 + bits, K, N, bits, gs, desc_act, M=4, bias=True)
    D = to_dev(L, dev)
    w16 = expected_weight(L)
    prep = prepare(D)
    for M in (1, 4, 2, 3, 1):
        plan = _lib.select_tiled(M, K, N, bits, gs)
        assert plan.kernel == _lib.KERNEL_TILED_DECODE and plan.split_k == 1
        tiles = N // 32
        halved = tiles if (2 * tiles <= 256 and -(-K // 64) >= 64) else tiles % 256
        assert plan.grid_x == tiles + halved and plan.workspace_bytes > 16384, "the plan does not halve its tiles"
        x = L["x"][:M].contiguous()
        want = expected_output(L, x=x, w16=w16)
        y = run_tiled(D, prep, x=x.to(dev), plan=plan)
        what = f"halved tiles int{bits} {K}x{N} M={M}"
        assert_close(y, want, what)
        if K >= 8192 and bits != 8:
            # The decode kernels multiply x with the codes exactly and apply scale and zero per group in fp32, so
            # what they compute is the product with the UNROUNDED weights scale * (q - zero); the reference rounds
            # every weight to fp16 first, a noise that grows with sqrt(K) and passes the tight bound at these
            # lengths.  Against the unrounded product the kernel is held to the rounding of y alone.
            assert_close(y, unrounded_output(L, x), what + " (against the unrounded weights)", rtol=1e-3, atol=1e-3)
        else:
            assert_tight(y, want, what)
        assert torch.equal(y, run_tiled(D, prep, x=x.to(dev), plan=plan)), f"{what}: two identical calls differ"


def _random_matmul_shapes():
    import random

    rnd = random.Random(20250)
    shapes = []
    for _ in range(48):
        bits = rnd.choice([2, 3, 4, 8])
        gs = rnd.choice([32, 64, 128, -1])
        K = 32 * rnd.randint(1, 100) if gs == -1 else gs * rnd.randint(1, 40)
        N = 32 * rnd.randint(1, 80)
        M = rnd.choice([rnd.randint(9, 32), rnd.randint(33, 64), rnd.randint(65, 128), rnd.randint(129, 300)])
        shapes.append((bits, K, N, gs, rnd.random() < 0.5, M))
    return shapes


@pytest.mark.parametrize("bits,K,N,gs,desc_act,M", _random_matmul_shapes())
def test_tiled_matmul_random_shapes(dev, bits, K, N, gs, desc_act, M):
    # the planner's own matmul plan (every block height, one to several row blocks, K whole or in ranges) on shapes
    # drawn at random with a fixed seed
    L = layer(9100 + K % 997 + N % 991, K, N, bits, gs, desc_act, M=M, bias=(M % 2 == 0))
    D = to_dev(L, dev)
    prep = prepare(D)
    plan = _lib.select_tiled(M, K, N, bits, gs)
    assert plan.kernel == _lib.KERNEL_TILED
    y = run_tiled(D, prep)
    what = (f"int{bits} {K}x{N} gs={gs} act={desc_act} M={M} ({plan.row_tiles} row tiles x {plan.m_blocks} blocks, "
            f"{plan.split_k} ranges of {plan.k_chunk} blocks per wave)")
    assert_close(y, expected_output(L), what)
    assert_tight(y, expected_output(L), what)


def _random_decode_shapes():
    import random

    rnd = random.Random(20240)
    shapes = []
    for _ in range(28):
        bits = rnd.choice([2, 3, 4, 8])
        gs = rnd.choice([32, 64, 128, 256, -1])
        unit = 32 if gs == -1 else gs
        kind = rnd.choice(["long-narrow", "tail-halved", "several-per-cu", "short"])
        if kind == "long-narrow":      # every tile in two halves
            K = unit * rnd.randint(-(-8192 // unit), -(-8192 // unit) + 40 * 32 // unit)
            N = 32 * rnd.randint(1, 24)
        elif kind == "tail-halved":    # up to 128 tiles past 256
            K = unit * rnd.randint(max(1, 256 // unit), 2048 // unit)
            N = 32 * rnd.randint(257, 384)
        elif kind == "several-per-cu":
            K = unit * rnd.randint(max(1, 128 // unit), 1024 // unit)
            N = 32 * rnd.randint(513, 700)
        else:
            K = unit * rnd.randint(1, max(1, 2048 // unit))
            N = 32 * rnd.randint(1, 160)
        shapes.append((bits, K, N, gs, rnd.random() < 0.6, rnd.randint(1, 4)))
    return shapes


@pytest.mark.parametrize("bits,K,N,gs,desc_act,M", _random_decode_shapes())
def test_tiled_decode_random_shapes(dev, bits, K, N, gs, desc_act, M):
    # the family's own decode plan (16-column units, a workgroup per tile, tail or all tiles halved, equal and
    # unequal halves, 4 to 16 waves along K) on shapes drawn at random with a fixed seed
    L = layer(9000 + K % 997 + N % 991, K, N, bits, gs, desc_act, M=M, bias=True)
    D = to_dev(L, dev)
    prep = prepare(D)
    plan = _lib.select_tiled(M, K, N, bits, gs)
    assert plan.kernel == _lib.KERNEL_TILED_DECODE
    y = run_tiled(D, prep, plan=plan)
    what = f"int{bits} {K}x{N} gs={gs} act={desc_act} M={M} (grid {plan.grid_x}, {plan.waves_k} waves, {plan.k_chunk} blocks)"
    assert_close(y, expected_output(L), what)
    if bits != 8:
        assert_close(y, unrounded_output(L, L["x"]), what + " (against the unrounded weights)", rtol=1e-3, atol=1e-3)
    else:
        assert_tight(y, expected_output(L), what)
    assert torch.equal(y, run_tiled(D, prep, plan=plan)), f"{what}: two identical calls differ"


DECODE_FULL = [
    ("c1-int4-4096x4096", 4, 4096, 4096, 128, False, [1, 2, 4]),
    ("c2-int3-4096x11008-act", 3, 4096, 11008, 128, True, [1, 2, 3]),
    ("int4-4096x11008-act", 4, 4096, 11008, 128, True, [1, 4]),
    ("c3-int4-11008x4096", 4, 11008, 4096, 128, False, [1, 2, 4]),
    ("int3-11008x4096-act", 3, 11008, 4096, 128, True, [1, 4]),
    ("c5-int3-9216x9216-act-g1", 3, 9216, 9216, -1, True, [1]),
    ("c5-int3-9216x36864-act-g1", 3, 9216, 36864, -1, True, [1]),
    ("c5-int3-36864x9216-act-g1", 3, 36864, 9216, -1, True, [1]),
    ("int8-4096x11008-act", 8, 4096, 11008, 128, True, [1, 4]),
    ("int2-4096x11008-act", 2, 4096, 11008, 128, True, [1, 3]),
    ("int8-11008x4096", 8, 11008, 4096, 128, False, [2]),
    ("int2-4096x4096-g64", 2, 4096, 4096, 64, False, [1]),
    # long K on wide layers: the family's own plan takes eight or sixteen waves along K
    ("int4-8192x8192-act", 4, 8192, 8192, 128, True, [1, 2]),
    ("int3-13824x5120-act", 3, 13824, 5120, 128, True, [1, 4]),
    ("int4-6656x17920", 4, 6656, 17920, 128, False, [2]),
]


@pytest.mark.parametrize("name,bits,K,N,gs,desc_act,Ms", DECODE_FULL, ids=[f[0] for f in DECODE_FULL])
def test_tiled_decode_full_size(dev, name, bits, K, N, gs, desc_act, Ms):
    L = layer(7300 + [f[0] for f in DECODE_FULL].index(name), K, N, bits, gs, desc_act, M=max(Ms))
    D = to_dev(L, dev)
    w16 = expected_weight(L)
    prep = prepare(D)
    for M in Ms:
        x = L["x"][:M].contiguous()
        want = expected_output(L, x=x, w16=w16)
        for plan in (_lib.select_tiled(M, K, N, bits, gs), tile_decode_plan(M, K, N, bits, gs),
                     cu_decode_plan(M, K, N, bits, gs)):
            if plan is None:
                continue
            y = run_tiled(D, prep, x=x.to(dev), plan=plan)
            what = f"decode {name} M={M} ({'cu' if plan.waves_n == 2 else 'tile'}, {plan.waves_k} waves)"
            assert_close(y, want, what)
            assert_tight(y, want, what)
            assert torch.equal(y, run_tiled(D, prep, x=x.to(dev), plan=plan)), f"{what}: two identical calls differ"


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("M", [2, 128])
def test_tiled_linearity_at_full_size(dev, bits, M):
    # size-independent properties on the tiled kernels at the benchmark's size (decode kernel with halved tiles,
    # pack pass + matmul): f(2 x) = 2 f(x) exactly, f(a + b) = f(a) + f(b) up to rounding, and the rows of a batch
    # equal the same rows computed alone
    K, N, gs = 4096, 11008, 128
    L = layer(905 + bits, K, N, bits, gs, True, M=M)
    # keep fp16 subnormals out of x: doubling must stay exact on every path, matrix cores included
    L["x"] = torch.where(L["x"].abs() < 1e-3, torch.zeros_like(L["x"]), L["x"])
    D = to_dev(L, dev)
    prep = prepare(D)
    x = D["x"]
    y = run_tiled(D, prep)
    y2 = run_tiled(D, prep, x=(x * 2).contiguous())
    normal = y.float().abs() >= 2.0 ** -13  # an fp16-subnormal output rounds on a fixed grid, not a relative one
    assert torch.equal(y2.float()[normal], (y.float() * 2)[normal])
    ysum = run_tiled(D, prep, x=(x[0:1] + x[1:2]).contiguous())
    assert_close(ysum, (y[0:1].float() + y[1:2].float()).cpu(), "additivity", rtol=2e-2, atol=2e-2)
    if M > 4:   # a row of the product depends on its own row of x only: the decode kernel gives the same row
        y1 = run_tiled(D, prep, x=x[5:6].contiguous())
        assert_tight(y1, y[5:6].cpu(), "row 5 alone against row 5 of the batch")


TILED_FULL = [
    ("c4-int4-4096x11008-act", 4, 4096, 11008, 128, True, [16, 64, 128, 256]),
    ("c4-int3-4096x11008-act", 3, 4096, 11008, 128, True, [16, 64, 128, 256]),
    ("c4-int4-11008x4096-act", 4, 11008, 4096, 128, True, [16, 64, 128, 256]),
    ("c4-int3-11008x4096-act", 3, 11008, 4096, 128, True, [16, 64, 128, 256]),
    ("c3-int4-4096x4096", 4, 4096, 4096, 128, False, [8, 1024]),
    ("c5-int3-9216x36864-act-g1", 3, 9216, 36864, -1, True, [32]),
    ("c5-int3-36864x9216-act-g1", 3, 36864, 9216, -1, True, [32, 64, 128, 256]),   # (K in ranges over two turns of the chip)
    ("int4-4096x4096-act", 4, 4096, 4096, 128, True, [48, 64, 100, 128, 192, 256]),    # (a narrow layer: shorter row blocks)
    ("int3-18432x4608-act", 3, 18432, 4608, 128, True, [64, 256]),
    ("int8-4096x11008-act", 8, 4096, 11008, 128, True, [16, 128, 256]),
    ("int2-4096x11008-act", 2, 4096, 11008, 128, True, [16, 128, 256]),
    ("int8-11008x4096", 8, 11008, 4096, 128, False, [64]),
    ("int2-11008x4096-act", 2, 11008, 4096, 128, True, [64]),
]


@pytest.mark.parametrize("name,bits,K,N,gs,desc_act,Ms", TILED_FULL, ids=[f[0] for f in TILED_FULL])
def test_tiled_full_size(dev, name, bits, K, N, gs, desc_act, Ms):
    L = layer(7200 + [f[0] for f in TILED_FULL].index(name), K, N, bits, gs, desc_act, M=max(Ms))
    D = to_dev(L, dev)
    w16 = expected_weight(L)
    prep = prepare(D)
    for M in Ms:
        x = L["x"][:M].contiguous()
        y = run_tiled(D, prep, x=x.to(dev))
        want = expected_output(L, x=x, w16=w16)
        assert_close(y, want, f"tiled {name} M={M}")
        assert_tight(y, want, f"tiled {name} M={M}")
        assert torch.equal(y, run_tiled(D, prep, x=x.to(dev))), f"tiled {name} M={M}: two identical calls differ"


def module_of(L, dev, **kw):
    q = QuantLinear(L["bits"], L["group_size"], L["K"], L["N"], L.get("bias") is not None, **kw)
    q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias") if L.get(k) is not None})
    return q.to(dev)


@pytest.mark.parametrize("bits", [3, 4])
@pytest.mark.parametrize("desc_act", [False, True])
def test_quantlinear_routes_prompt_sizes_to_the_tiled_copy(dev, bits, desc_act):
    K, N, gs = 1024, 416, 128
    L = layer(1800 + bits, K, N, bits, gs, desc_act, M=150, bias=True)
    q = module_of(L, dev)
    assert q._tiled is None
    x = L["x"].to(dev)
    y12 = q(x[:12])                                # 9..16 rows: mostly on the checkpoint layout (or its sorted copy)
    assert (q._tiled is None) == (_lib.select_route(12, K, N, bits, gs, desc_act).copy != _lib.ROUTE_TILED)
    y40, y150, y2, y8 = q(x[:40]), q(x), q(x[:2]), q(x[:8])   # prompt sizes, and the decode sizes (up to eight rows)
    assert q._tiled is not None and q._tiled[1] is not None
    want = expected_output(L)
    for y, M in ((y2, 2), (y8, 8), (y12, 12), (y40, 40), (y150, 150)):
        assert_close(y, want[:M], f"module, {M} rows")
        assert_tight(y, want[:M], f"module, {M} rows")
    # the same numbers (to the tight bound) from the checkpoint's own tensors
    q.tile_for_prefill = False
    assert_tight(q(x[:40]), y40.cpu(), "module, tiled against unprepared")
    q.tile_for_prefill = True
    # new weights invalidate the copy
    L2 = layer(1810 + bits, K, N, bits, gs, desc_act, M=40, bias=True)
    q.load_state_dict({k: L2[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
    assert_close(q(L2["x"].to(dev)), expected_output(L2), "module after reload")
    # a layer the format does not cover (groups of 16 channels) keeps working
    L3 = layer(1820, 256, 64, 4, 16, False, M=40)
    q3 = module_of(L3, dev)
    assert_close(q3(L3["x"].to(dev)), expected_output(L3), "module, uncovered by the format")
    assert q3.route(40) == "plain" and not q3.compact() and q3._tiled[1] is None


@pytest.mark.parametrize("bits", [2, 8])
@pytest.mark.parametrize("desc_act", [False, True])
def test_quantlinear_runs_2_and_8_bits_fused_on_the_tiled_copy(dev, bits, desc_act):
    """2- and 8-bit layers have no kernels on the checkpoint layout: every row count below the switch to the
    library GEMM runs on the tiled copy; without it (or above the switch) the layer is dequantised."""
    K, N, gs = 1024, 416, 128
    L = layer(1850 + bits, K, N, bits, gs, desc_act, M=150, bias=True)
    q = module_of(L, dev, kernel_switch_threshold=128)
    x = L["x"].to(dev)
    want = expected_output(L)
    for M in (1, 3, 8, 40, 127):
        assert q.route(M) == "tiled"
        y = q(x[:M])
        assert_close(y, want[:M], f"module, {M} rows")
        assert_tight(y, want[:M], f"module, {M} rows")
    assert q.route(150) == "library"
    assert_close(q(x), want, "module, 150 rows (library)")
    off = module_of(L, dev, tile_for_prefill=False)
    assert off.route(1) == "library" and off._tiled is None
    assert_close(off(x[:3]), want[:3], "module without the tiled copy")
    assert q.compact() and q.route(150) == "tiled"
    assert_tight(q(x), want, "compact module, 150 rows")
    assert torch.equal(q.dequantize().cpu().view(torch.int16), expected_weight(L).view(torch.int16))


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("desc_act", [False, True])
def test_quantlinear_compact_keeps_one_copy(dev, bits, desc_act):
    K, N, gs = 1024, 416, 128
    L = layer(1900 + bits, K, N, bits, gs, desc_act, M=300, bias=True)
    q = module_of(L, dev, kernel_switch_threshold=256)
    assert q.compact() and q.compact()
    assert q.qweight.numel() == 0 and q.qzeros.numel() == 0 and q.scales.numel() == 0 and q._sorted is None
    x = L["x"].to(dev)
    want = expected_output(L)
    for M in (1, 3, 8, 40, 300):                   # 300 rows: above the threshold, still the tiled kernels
        y = q(x[:M])
        assert_close(y, want[:M], f"compact module, {M} rows")
        assert_tight(y, want[:M], f"compact module, {M} rows")
    assert torch.equal(q.dequantize().cpu().view(torch.int16), expected_weight(L).view(torch.int16))
    q = q.to(dev)                                  # moving the module keeps the copy
    assert_close(q(x[:40]), want[:40], "compact module after .to()")
    # a gradient for x needs the copy for it, made before the checkpoint tensors went: without one the layer says so
    # instead of forming W through a K-row product
    xg = x[:4].clone().requires_grad_(True)
    with pytest.raises(RuntimeError, match="prepare_transposed"):
        q(xg).float().sum().backward()
    q2 = module_of(L, dev)
    assert q2.prepare_transposed() is not None and q2.compact()
    xg = x[:4].clone().requires_grad_(True)
    q2(xg).float().sum().backward()               # (adapters on top of frozen layers)
    assert xg.grad is not None and xg.grad.shape == xg.shape


@pytest.mark.parametrize("bits", [3, 4])
def test_long_prompts_run_fused_on_the_tiled_kernels(dev, bits):
    """1024 and 4096 rows stay on the fused path when the switch to the library GEMM is off (and always on a
    compact layer): the matmul kernel walks the row blocks itself."""
    K, N, gs = 512, 192, 128
    L = layer(2000 + bits, K, N, bits, gs, True, M=4096, bias=True)
    q = module_of(L, dev, kernel_switch_threshold=None)
    x = L["x"].to(dev)
    want = expected_output(L)
    for M in (1024, 4096):
        assert q.route(M) == "tiled"
        y = q(x[:M])
        assert_close(y, want[:M], f"module, {M} rows")
        assert_tight(y, want[:M], f"module, {M} rows")
    q.kernel_switch_threshold = 1024
    assert q.route(1024) == "library" and q.route(1023) == "tiled"
    assert q.compact() and q.route(4096) == "tiled"
    assert_tight(q(x), want, "compact module, 4096 rows")


@pytest.mark.parametrize("compact", [False, True])
def test_quantlinear_copies_after_it_has_served_calls(dev, compact):
    """copy.deepcopy and pickle of a module whose routes are populated (bound C++ launch objects, closures over its
    tensors): the copy has its own tensors, decides its routes again and gives the same numbers."""
    import copy
    import pickle

    K, N, gs = 1024, 416, 128
    L = layer(1900, K, N, 4, gs, True, M=40, bias=True)
    q = module_of(L, dev)
    if compact:
        assert q.compact()
    x = L["x"].to(dev)
    y1, y40 = q(x[:1]), q(x)
    assert q._routes
    for clone in (copy.deepcopy(q), pickle.loads(pickle.dumps(q))):
        assert clone._routes == {} and clone._compact == compact
        if compact:
            assert clone._tiled[1][0].data_ptr() != q._tiled[1][0].data_ptr()
        else:
            assert clone.qweight.data_ptr() != q.qweight.data_ptr()
        assert torch.equal(clone(x[:1]), y1) and torch.equal(clone(x), y40)
        # the copy computes on its own weights: changing the original's does not reach it
        if not compact:
            q.qweight.zero_()
            assert torch.equal(clone(x), y40)
            q.load_state_dict({k: L[k] for k in ("qweight", "qzeros", "scales", "g_idx", "bias")})
            q.to(dev)


@pytest.mark.parametrize("bits,K,N,gs,desc_act", [(4, 1024, 416, 128, True), (3, 4096, 4096, 128, False),
                                                   (4, 2048, 8224, 128, True), (3, 1024, 160, -1, True)])
def test_quantlinear_takes_the_route_the_library_names(dev, bits, K, N, gs, desc_act):
    """QuantLinear asks gptq_hip_select_route which copy a call runs on; the path it reports is that answer."""
    L = layer(1910 + bits, K, N, bits, gs, desc_act, M=1)
    q = module_of(L, dev)
    for M in (1, 2, 4, 8, 16, 17, 64, 128, 300, 700, 1100, 1200):
        r = _lib.select_route(M, K, N, bits, gs, desc_act and gs != -1)
        assert q.route(M) == _lib.ROUTE_NAMES[r.copy], (M, q.route(M), r.copy)
    # swapping a buffer behind the module's back (what offload hooks do) makes it decide again, on the new tensor
    x = torch.randn(3, K, dtype=torch.float16, device=dev)
    before = q(x)
    q._buffers["qweight"] = torch.zeros_like(q.qweight)
    q._g_state = None
    after = q(x)
    assert not torch.equal(before, after)


@pytest.mark.parametrize("bits", [2, 3, 4, 8])
@pytest.mark.parametrize("K,N,gs", [(32, 32, 32), (160, 96, -1), (384, 64, 64), (1024, 416, 32), (2048, 1056, 256),
                                    (4096, 352, 128), (11008, 256, 128), (4096, 11008, 128)])
@pytest.mark.parametrize("M", [5, 6, 8])
def test_tiled_decode_five_to_eight_rows(dev, bits, K, N, gs, M):
    """The decode kernel with two sets of four rows (5 to 8 rows): against the oracle to the contract's bound and the
    tight one, twice with equal results, with and without an activation order, halved tiles and long K included."""
    for desc_act in (False, True):
        L = layer(1700 + K + M, K, N, bits, gs, desc_act, M=M, bias=(M % 2 == 0))
        D = to_dev(L, dev)
        plan = _lib.select_tiled(M, K, N, bits, gs, decode=True)
        assert plan.kernel == _lib.KERNEL_TILED_DECODE and plan.row_tiles == 8 and plan.waves_k in (4, 8)
        prep = prepare(D)
        want = expected_output(L)
        y = run_tiled(D, prep, plan=plan)
        assert_close(y, want, f"decode, two row sets: bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
        assert_tight(y, want, f"decode, two row sets: bits={bits} K={K} N={N} gs={gs} M={M} act={desc_act}")
        assert torch.equal(y, run_tiled(D, prep, plan=plan)), "two identical calls differ"
